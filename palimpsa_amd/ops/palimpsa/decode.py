"""Single-token decode with the per-call host work done once.

``fused_recurrent_palimpsa`` validates, normalises and allocates on every call (about 35 us of Python
for a 5 us kernel at small batch).  A serving loop that keeps its state tensors alive can bind them
once: ``DecodeStep`` checks shapes and dtypes at construction, fills the C structs once and per step
only issues ``pal_recurrent_fwd`` on the current stream.  The state ``(mu, I)`` is updated in place
(the kernel reads a state entry and writes it back from the same thread), the output buffer is
reused, nothing is allocated per step, so the step can also be recorded into a HIP graph.
Same kernel and same arithmetic as ``fused_recurrent_palimpsa`` with ``T = 1``
(reference call site: palimpsa/layers/palimpsa.py:317, mode 'fused_recurrent').
"""
from __future__ import annotations

import ctypes as C
from typing import Optional

import torch

from ... import _lib as L
from . import _common as cm


class DecodeStep:
    """Bound decode step for fixed shapes: ``B`` sequences, ``H`` heads, head dims ``dk``, ``dv``.

    ``rows_dtype`` is the dtype of q, k, v, b (bf16 or fp32); gt, g, Ip and the states are fp32.
    ``dk`` must be one of the head dims the token-serial kernel is compiled for and ``dv`` a
    multiple of 16 (no padding here: a server lays its state out once).  ``tokens`` > 1 makes a step
    consume that many tokens per sequence (blocked or speculative decode): the state stays in registers
    over the block and is read and written once.  ``mu_dtype=torch.bfloat16`` keeps the mean state in bf16
    between steps (``bind`` then takes a bf16 ``mu``; ``I`` stays fp32): 12 instead of 16 bytes of traffic per
    state entry and step, at a rounding error of 2^-9 relative per step that decays with the forgetting
    factor (``mu_to_cache`` / ``mu_from_cache`` convert to and from the fp32 pair the layers hand around)."""

    def __init__(self, B: int, H: int, dk: int, dv: int, device, rows_dtype=torch.bfloat16,
                 scale: Optional[float] = None, output_uncertainty: bool = False, tokens: int = 1,
                 mu_dtype=torch.float32):
        dev = torch.device(device)
        if dev.type != "cuda":
            raise RuntimeError("palimpsa_amd runs on an AMD GPU only; there is no CPU fallback")
        if dev.index is None:
            dev = torch.device("cuda", torch.cuda.current_device())
        if cm.padded_dk(dk, True) != dk or cm.padded_dv(dv) != dv:
            raise ValueError(f"dk must be one of {L.RECURRENT_DK} and dv a multiple of 16; got dk={dk}, dv={dv}")
        if rows_dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("rows_dtype must be torch.bfloat16 or torch.float32")
        if not isinstance(tokens, int) or tokens < 1:
            raise ValueError(f"tokens must be a positive int, got {tokens!r}")
        if mu_dtype not in (torch.float32, torch.bfloat16):
            raise ValueError("mu_dtype must be torch.float32 or torch.bfloat16")
        self.tokens = tokens
        self.mu_dtype = mu_dtype
        self.B, self.H, self.dk, self.dv, self.device, self.rows_dtype = B, H, dk, dv, dev, rows_dtype
        self.o = torch.empty(B, tokens, H, dv, dtype=rows_dtype, device=dev)
        self.o_var = torch.empty(B, tokens, H, dv, dtype=torch.float32, device=dev) if output_uncertainty else None
        flags = L.PAL_FLAG_HAS_INIT | L.PAL_FLAG_STORE_FINAL | (L.PAL_FLAG_HAS_VAR if output_uncertainty else 0)
        if mu_dtype == torch.bfloat16:
            flags |= L.PAL_FLAG_STATE_MU_BF16
        self._dims = L.PalDims(batch=B, seq_len=tokens, n_seqs=B, n_heads=H, dk=dk, dv=dv, total_chunks=0,
                               dtype=cm._pal_dtype(rows_dtype), gate_dtype=L.PAL_DTYPE_F32, var_dtype=L.PAL_DTYPE_F32,
                               flags=flags, scale=float(dk ** -0.5 if scale is None else scale))
        self._tens = L.PalFwdTensors(o=cm._ptr(self.o), o_var=cm._ptr(self.o_var))
        self._fn = L.load().pal_recurrent_fwd
        self._row_shape = (B, tokens, H)

    def _check(self, name, x, shape, dtype):
        if tuple(x.shape) != shape or x.dtype != dtype or x.device != self.device or not x.is_contiguous():
            raise ValueError(f"{name}: expected contiguous {dtype} {shape} on {self.device}, "
                             f"got {x.dtype} {tuple(x.shape)} on {x.device}")

    def bind(self, q, k, v, b, gt, g, Ip, mu, I) -> "DecodeStep":
        """Check the tensors once and remember their addresses; later steps reuse them (write the next
        token's rows into the same tensors) or pass new ones to ``step``."""
        rs = self._row_shape
        self._check("q", q, rs + (self.dk,), self.rows_dtype)
        self._check("k", k, rs + (self.dk,), self.rows_dtype)
        self._check("v", v, rs + (self.dv,), self.rows_dtype)
        self._check("b", b, rs + (self.dv,), self.rows_dtype)
        self._check("gt", gt, rs, torch.float32)
        self._check("g", g, (self.H,), torch.float32)
        self._check("Ip", Ip, (self.H,), torch.float32)
        self._check("mu", mu, (self.B, self.H, self.dv, self.dk), self.mu_dtype)
        self._check("I", I, (self.B, self.H, self.dv, self.dk), torch.float32)
        t = self._tens
        t.q, t.k, t.v, t.b, t.gt = q.data_ptr(), k.data_ptr(), v.data_ptr(), b.data_ptr(), gt.data_ptr()
        t.g, t.Ip = g.data_ptr(), Ip.data_ptr()
        t.init_mu = t.final_mu = mu.data_ptr()
        t.init_I = t.final_I = I.data_ptr()
        self._keep = (q, k, v, b, gt, g, Ip, mu, I)
        return self

    def step(self, stream: Optional[int] = None) -> torch.Tensor:
        """One token (``tokens`` of them) for every sequence from the bound tensors; returns the (reused) output
        buffer ``[B,tokens,H,dv]``.  ``stream`` is a raw HIP stream handle; default: torch's current stream."""
        if stream is None:
            rc = self._fn(self._dims, self._tens, cm.current_stream_ptr(self.device))
        else:
            rc = self._fn(self._dims, self._tens, C.c_void_p(stream))
        if rc:
            L.check(rc, "pal_recurrent_fwd")
        return self.o


def mu_to_cache(mu: torch.Tensor) -> torch.Tensor:
    """fp32 mean state ``[N,H,dv,dk]`` (what the entry points return) -> the bf16 cache form of ``DecodeStep``."""
    return mu.to(torch.bfloat16).contiguous()


def mu_from_cache(mu: torch.Tensor) -> torch.Tensor:
    """bf16 cache form -> the fp32 mean state the entry points take as ``initial_mu_state``."""
    return mu.to(torch.float32).contiguous()
