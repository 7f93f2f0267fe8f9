"""Host-side plumbing shared by the two operator entry points: dtype and layout
normalisation, zero-padding of head dims the kernels are not compiled for, and
filling the C structs.  PyTorch is used for device memory and streams only."""
from __future__ import annotations

import ctypes as C
import weakref
from dataclasses import dataclass
from typing import Optional

import torch
import torch.nn.functional as F

from ... import _lib as L


def no_compile(fn):
    """Keep torch.compile from tracing into an entry point: the work happens in ctypes calls that a tracer cannot
    follow, so the call is left as an opaque eager region (a graph break) instead of being probed and warned about."""
    disable = getattr(getattr(torch, "compiler", None), "disable", None)
    return disable(fn) if disable is not None else fn


def _require_gpu(*tensors) -> torch.device:
    dev = tensors[0].device
    if dev.type != "cuda":
        raise RuntimeError(
            "palimpsa_amd runs on an AMD GPU only (hand-written HIP kernels for gfx950); "
            f"got a tensor on '{dev}'. There is no CPU fallback: use palimpsa_ref for a CPU evaluation.")
    for t in tensors:
        if t is not None and t.device != dev:
            raise ValueError(f"all tensors must be on {dev}, found {t.device}")
    return dev


def _round_up(x: int, m: int) -> int:
    return (x + m - 1) // m * m


def padded_dk(dk: int, recurrent: bool) -> int:
    if dk > 256:
        raise ValueError(f"head dim {dk} > 256 is not supported")
    if recurrent:
        for c in L.RECURRENT_DK:
            if c >= dk:
                return c
    return _round_up(dk, 16)


def padded_dv(dv: int) -> int:
    if dv > 256:
        raise ValueError(f"value head dim {dv} > 256 is not supported")
    return _round_up(dv, 16)


def _pal_dtype(dt: torch.dtype) -> int:
    return L.PAL_DTYPE_BF16 if dt == torch.bfloat16 else L.PAL_DTYPE_F32


@dataclass
class Prepared:
    """Kernel-ready views of the operator inputs (contiguous, padded, supported dtypes)."""
    q: torch.Tensor
    k: torch.Tensor
    v: torch.Tensor
    b: torch.Tensor
    gt: torch.Tensor
    g: torch.Tensor
    Ip: torch.Tensor
    init_mu: Optional[torch.Tensor]
    init_I: Optional[torch.Tensor]
    cu_seqlens: Optional[torch.Tensor]
    dk: int          # logical dims
    dv: int
    dk_p: int        # padded dims handed to the kernels
    dv_p: int
    n_seqs: int
    compute_dtype: torch.dtype


def prepare_inputs(q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state, cu_seqlens, recurrent: bool) -> Prepared:
    dev = _require_gpu(q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state)
    if q.dim() != 4 or k.shape != q.shape or v.dim() != 4 or b.shape != v.shape or v.shape[:2] != q.shape[:2]:
        raise ValueError("expected q,k [B,T,Hq,dk] and v,b [B,T,H,dv] (Hq = H, or a divisor of H)")
    B, T, H, dv = v.shape
    Hq, dk = q.shape[2], q.shape[3]
    # q and k may carry fewer heads than v: a group of H / Hq value heads then shares one q/k head, which is what
    # the reference layers obtain by repeating heads before the call (layers/meta_mamba2.py:281-282,
    # layers/palimpsa.py:266-267); the kernels index the shared rows instead
    if Hq < 1 or H % Hq != 0:
        raise ValueError(f"the {Hq} heads of q, k must divide the {H} heads of v, b")
    if tuple(gt.shape) != (B, T, H):
        raise ValueError(f"gt must be [B,T,H]={(B, T, H)}, got {tuple(gt.shape)}")
    if g.numel() != H or Ip.numel() != H:
        raise ValueError("g and Ip must have one entry per head")
    # one element type for q,k,v,b: bf16 stays bf16, everything else computes from fp32 rows
    cd = torch.bfloat16 if all(x.dtype == torch.bfloat16 for x in (q, k, v, b)) else torch.float32
    q, k, v, b = [x.to(cd).contiguous() for x in (q, k, v, b)]
    if gt.dtype not in (torch.float32, torch.bfloat16):
        gt = gt.float()
    gt = gt.contiguous()
    if gt.data_ptr() % 4:       # a bf16 view that starts on an odd element: the kernels fetch gates as aligned words
        gt = gt.clone()
    g = g.reshape(H).float().contiguous()
    Ip = Ip.reshape(H).float().contiguous()
    n_seqs = B
    if cu_seqlens is not None:
        n_seqs = int(cu_seqlens.numel()) - 1
        cu_seqlens = cu_seqlens.to(device=dev, dtype=torch.int32).contiguous()
    dk_p, dv_p = padded_dk(dk, recurrent), padded_dv(dv)
    if dk_p != dk:
        q = F.pad(q, (0, dk_p - dk))
        k = F.pad(k, (0, dk_p - dk))
    if dv_p != dv:
        v = F.pad(v, (0, dv_p - dv))
        b = F.pad(b, (0, dv_p - dv))
    if (initial_mu_state is None) != (initial_I_state is None):
        # the layer may hand over a bare recurrent state (layers/palimpsa.py:305-306 of the
        # reference); the kernels need both halves
        raise ValueError("initial_mu_state and initial_I_state must be given together")
    if initial_mu_state is not None:
        exp = (n_seqs, H, dv, dk)
        if tuple(initial_mu_state.shape) != exp or tuple(initial_I_state.shape) != exp:
            raise ValueError(f"Initial states mismatch: expected {exp}, got "
                             f"{tuple(initial_mu_state.shape)} / {tuple(initial_I_state.shape)}")
        initial_mu_state = initial_mu_state.float().contiguous()
        initial_I_state = initial_I_state.float().contiguous()
        if dk_p != dk or dv_p != dv:
            pad = (0, dk_p - dk, 0, dv_p - dv)
            initial_mu_state = F.pad(initial_mu_state, pad, value=0.0)
            initial_I_state = F.pad(initial_I_state, pad, value=1.0)
    return Prepared(q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state, cu_seqlens,
                    dk, dv, dk_p, dv_p, n_seqs, cd)


# chunk bookkeeping of the packed batches seen last, per cu_seqlens tensor object: the layers of a model hand the
# same tensor to every operator call of a step, so the device-to-host copy (a stream synchronisation) and the
# table happen once per step instead of once per layer
_chunk_meta_cache: dict = {}
_CHUNK_META_CACHE_MAX = 8


def chunk_meta(cu_seqlens: torch.Tensor, total_tokens: int, device: torch.device):
    """cu_seqlens (any int dtype/device) -> (packed int32 metadata on ``device``, total_chunks).

    The metadata is ``[N+1]`` cumulative chunk counts followed by ``[total_chunks,4]`` rows (sequence, first
    token, length, index in sequence).  Raises ValueError unless cu_seqlens starts at 0, never decreases and
    ends at ``total_tokens`` (the kernels take sequence bounds from it).  Results are kept per tensor object
    (weakly referenced, invalidated by in-place writes through torch), not per address: a new tensor that
    reuses the memory of a dead one is looked at again.  A host tensor is also compared element by element with
    the copy taken when its entry was made (its memory may be shared with an array that a loader rewrites without
    torch noticing).  For a device tensor the entry relies on torch's version counter: a kernel or extension that
    writes through ``data_ptr()`` must call ``invalidate_chunk_meta()`` (or hand over a new tensor)."""
    key = id(cu_seqlens)
    hit = _chunk_meta_cache.get(key)
    if hit is not None:
        ref, version, tokens, dev, packed, total, host_copy = hit
        if (ref() is cu_seqlens and version == cu_seqlens._version and tokens == total_tokens and dev == device
                and (host_copy is None or torch.equal(cu_seqlens.detach().to(torch.int64), host_copy))):
            return packed, total
    if cu_seqlens.dim() != 1 or cu_seqlens.numel() < 2:
        raise ValueError(f"cu_seqlens must be a 1-D tensor of at least two entries, got shape {tuple(cu_seqlens.shape)}")
    cu_host = cu_seqlens.detach().to("cpu", torch.int64).numpy()
    if int(cu_host[0]) != 0 or bool((cu_host[1:] < cu_host[:-1]).any()) or int(cu_host[-1]) != int(total_tokens):
        raise ValueError(
            "cu_seqlens must start at 0, be non-decreasing and end at the token count "
            f"({total_tokens}); got first={int(cu_host[0])}, last={int(cu_host[-1])}, "
            f"decreasing={bool((cu_host[1:] < cu_host[:-1]).any())}")
    table, offsets = L.build_chunk_table(cu_host)
    packed = torch.cat([torch.from_numpy(offsets), torch.from_numpy(table.reshape(-1))]).to(torch.int32).to(device)
    total = int(table.shape[0])
    if len(_chunk_meta_cache) >= _CHUNK_META_CACHE_MAX:
        _chunk_meta_cache.pop(next(iter(_chunk_meta_cache)))
    try:
        ref = weakref.ref(cu_seqlens, lambda _r, k=key: _chunk_meta_cache.pop(k, None))
    except TypeError:
        return packed, total
    host_copy = torch.from_numpy(cu_host).clone() if cu_seqlens.device.type == "cpu" else None
    _chunk_meta_cache[key] = (ref, cu_seqlens._version, int(total_tokens), device, packed, total, host_copy)
    return packed, total


def invalidate_chunk_meta() -> None:
    """Forget the chunk bookkeeping kept per cu_seqlens tensor (for callers that rewrite a device cu_seqlens
    tensor behind torch's back)."""
    _chunk_meta_cache.clear()


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def make_dims(p: Prepared, scale: float, flags: int, total_chunks: int = 0, var_dtype: torch.dtype = torch.float32,
              mode_flags: Optional[int] = None) -> L.PalDims:
    """``mode_flags``: the knob bits (state-pass form, fp32 treatment) to use instead of the current settings, for a
    backward that has to run in the mode its forward ran in."""
    B, T, H, _ = p.v.shape
    return L.PalDims(batch=B, seq_len=T, n_seqs=p.n_seqs, n_heads=H, dk=p.dk_p, dv=p.dv_p,
                     total_chunks=total_chunks, dtype=_pal_dtype(p.compute_dtype),
                     gate_dtype=_pal_dtype(p.gt.dtype), var_dtype=_pal_dtype(var_dtype),
                     flags=flags | (L.state_pass_flags() if mode_flags is None else int(mode_flags)), scale=float(scale),
                     n_qk_heads=p.q.shape[2])


def make_fwd_tensors(p: Prepared, o, o_var, final_mu, final_I, chunk_table=None, chunk_offsets=None,
                     chunk_mu=None, chunk_I=None) -> L.PalFwdTensors:
    return L.PalFwdTensors(
        q=_ptr(p.q), k=_ptr(p.k), v=_ptr(p.v), b=_ptr(p.b), gt=_ptr(p.gt), g=_ptr(p.g), Ip=_ptr(p.Ip),
        o=_ptr(o), o_var=_ptr(o_var), init_mu=_ptr(p.init_mu), init_I=_ptr(p.init_I),
        final_mu=_ptr(final_mu), final_I=_ptr(final_I), cu_seqlens=_ptr(p.cu_seqlens),
        chunk_table=_ptr(chunk_table), chunk_offsets=_ptr(chunk_offsets),
        chunk_mu=_ptr(chunk_mu), chunk_I=_ptr(chunk_I))


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream_ptr(dev: torch.device):
    """Handle of torch's current stream on ``dev`` for the C ABI (the raw accessor saves ~20 us of host time
    per call over constructing a torch.cuda.Stream object)."""
    if _raw_stream is not None:
        return C.c_void_p(_raw_stream(dev.index if dev.index is not None else torch.cuda.current_device()))
    return C.c_void_p(torch.cuda.current_stream(dev).cuda_stream)


def unpad_state(x: Optional[torch.Tensor], p: Prepared):
    if x is None or (p.dk_p == p.dk and p.dv_p == p.dv):
        return x
    return x[:, :, :p.dv, :p.dk].contiguous()


def unpad_last(x: Optional[torch.Tensor], n: int):
    if x is None or x.shape[-1] == n:
        return x
    return x[..., :n].contiguous()
