"""CPU restatement of the Palimpsa naive recurrence (TEST INFRASTRUCTURE ONLY).

This file is the checker the HIP kernels are compared against.  It is never
imported by the shipped package: the product path must fail loudly when the
HIP extension is missing rather than fall back to this code.

What it restates (all citations are into the reference repository):

* values: ``palimpsa_ref`` in
  palimpsa/ops/palimpsa/chunk_palimpsa_forgetting_scalar.py:669-725
  (per-token loop: M = v k^T + f*mu_pre*I_pre  (:712),
  I = b (k*k)^T + (1-f)*Ip + f*I_pre (:713), mu = M/I (:714),
  y = mu q*scale (:717), y_var = (1/I) (q*scale)^2 (:718)).
* state format (mu, I), fp32, [N, H, dv, dk]:
  palimpsa/ops/palimpsa/fused_recurrent_palimpsa.py:84-96, :145-154.
* default state (mu, I) = (0, Ip): chunk...py:702-704, :139-140.
* varlen = independent documents, each starting from its own initial state:
  chunk...py:96-108, fused...py:51-55, and the test topology of
  palimpsa/check_palimpsa.py:157-179.
* ``o_var`` has two conventions in the reference: the naive loop scales q
  before squaring (scale**2, chunk...py:709,:718) while both Triton kernels
  multiply by scale once (chunk...py:204, fused...py:136).  They agree at
  scale == 1, the only value the reference's own check uses
  (check_palimpsa.py:95-100).  ``var_scale_power`` selects which one.

Pinning status: every function here is pinned by tests/test_oracle_pins.py
against closed forms (T=1, b==0 gated-linear-attention as a masked float64
matmul, gt==0 cumulative sums, infinite decay, scalar recurrences), a float64
brute-force direct summation, invariants (split/resume, varlen == per-document
runs, linearity in v) and ``torch.autograd.gradcheck``.  The reference ships no
golden vectors for this path (it has no tests directory), so none are used.
``chunk_offsets`` / ``build_chunk_table`` restate integer helpers of the
un-vendored third-party package ``fla`` (unpinned version; call sites
chunk...py:633-638); for those the reference holds no stored values either:
they are re-derived from call-site semantics and are "parity unpinned"
against the third-party code itself.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import numpy as np
import torch


# --------------------------------------------------------------------------
# forward recurrence (torch, differentiable, fp32 or fp64)
# --------------------------------------------------------------------------
def _run_one_batch(q, k, v, b, gt, g, Ip, mu0, I0, scale, var_scale_power, want_var):
    """One fixed-length batch [B, T, H, *]; follows chunk...py:697-725."""
    B, T, H, DV = v.shape
    DK = k.shape[-1]
    dt = v.dtype
    if mu0 is None:
        mu_pre = torch.zeros(B, H, DV, DK, dtype=dt)
        I_pre = Ip.view(1, H, 1, 1).expand(B, H, DV, DK)
    else:
        mu_pre, I_pre = mu0, I0
    ys, yvars = [], []
    Ipb = Ip.view(1, H, 1, 1)
    for t in range(T):
        f = torch.exp(-gt[:, t, :] * g.view(1, H)).view(B, H, 1, 1)
        kt = k[:, t].unsqueeze(-2)            # [B,H,1,DK]
        M = v[:, t].unsqueeze(-1) * kt + f * mu_pre * I_pre
        I = b[:, t].unsqueeze(-1) * (kt * kt) + (1.0 - f) * Ipb + f * I_pre
        mu = M / I
        qt = q[:, t]
        ys.append(scale * torch.einsum("bhdn,bhn->bhd", mu, qt))
        if want_var:
            yvars.append((scale ** var_scale_power) * torch.einsum("bhdn,bhn->bhd", 1.0 / I, qt * qt))
        mu_pre, I_pre = mu, I
    y = torch.stack(ys, dim=1) if T > 0 else torch.zeros(B, 0, H, DV, dtype=dt)
    yv = torch.stack(yvars, dim=1) if (want_var and T > 0) else None
    return y, yv, mu_pre, I_pre


def palimpsa_recurrence(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    b: torch.Tensor,
    gt: torch.Tensor,
    g: torch.Tensor,
    Ip: torch.Tensor,
    initial_mu_state: Optional[torch.Tensor] = None,
    initial_I_state: Optional[torch.Tensor] = None,
    scale: Optional[float] = None,
    cu_seqlens: Optional[Sequence[int]] = None,
    output_uncertainty: bool = False,
    var_scale_power: int = 1,
    compute_dtype: torch.dtype = torch.float32,
):
    """Naive token-serial Palimpsa recurrence on the CPU.

    Shapes: q,k [B,T,H,dk]; v,b [B,T,H,dv]; gt [B,T,H]; g,Ip [H];
    states [N,H,dv,dk] with N = B, or the number of documents when
    ``cu_seqlens`` (length N+1, requires B == 1) is given.

    Returns ``(o, o_var_or_None, final_mu, final_I)`` in ``compute_dtype``.
    Differentiable w.r.t. every floating input.
    """
    cd = compute_dtype
    q, k, v, b, gt, g, Ip = [x.to(cd) for x in (q, k, v, b, gt, g, Ip)]
    if initial_mu_state is not None:
        initial_mu_state = initial_mu_state.to(cd)
        initial_I_state = initial_I_state.to(cd)
    if scale is None:
        scale = q.shape[-1] ** -0.5      # chunk...py:693-694
    if cu_seqlens is None:
        return _run_one_batch(q, k, v, b, gt, g, Ip, initial_mu_state, initial_I_state,
                              scale, var_scale_power, output_uncertainty)
    cu = [int(x) for x in cu_seqlens]
    if q.shape[0] != 1:
        raise ValueError("varlen needs batch size 1")
    ys, yvs, fmu, fI = [], [], [], []
    for n in range(len(cu) - 1):
        s, e = cu[n], cu[n + 1]
        mu0 = None if initial_mu_state is None else initial_mu_state[n:n + 1]
        I0 = None if initial_I_state is None else initial_I_state[n:n + 1]
        y, yv, m_, i_ = _run_one_batch(q[:, s:e], k[:, s:e], v[:, s:e], b[:, s:e], gt[:, s:e],
                                       g, Ip, mu0, I0, scale, var_scale_power, output_uncertainty)
        ys.append(y)
        yvs.append(yv)
        fmu.append(m_)
        fI.append(i_)
    y = torch.cat(ys, dim=1)
    yv = torch.cat(yvs, dim=1) if output_uncertainty else None
    return y, yv, torch.cat(fmu, dim=0), torch.cat(fI, dim=0)


# --------------------------------------------------------------------------
# float64 brute force: direct summation, no recurrence (numpy, tiny inputs)
# --------------------------------------------------------------------------
def direct_sum_states(k, v, b, gt, g, Ip, mu0=None, I0=None):
    """States of ONE (sequence, head) by explicit double sums.

    k [T,dk], v,b [T,dv], gt [T], scalars g, Ip.  Returns (M, I) of shape
    [T, dv, dk] with
      M_t = sum_{s<=t} (prod_{r=s+1..t} f_r) v_s k_s^T + (prod_{r<=t} f_r) mu0*I0
      I_t = Ip + sum_{s<=t} (prod ...) b_s (k_s*k_s)^T + (prod_{r<=t} f_r)(I0-Ip)
    which is what unrolling chunk...py:712-713 gives.
    """
    k = np.asarray(k, np.float64)
    v = np.asarray(v, np.float64)
    b = np.asarray(b, np.float64)
    gt = np.asarray(gt, np.float64)
    T, dk = k.shape
    dv = v.shape[1]
    f = np.exp(-gt * float(g))
    M0 = np.zeros((dv, dk)) if mu0 is None else np.asarray(mu0, np.float64) * np.asarray(I0, np.float64)
    J0 = np.zeros((dv, dk)) if I0 is None else np.asarray(I0, np.float64) - float(Ip)
    M = np.zeros((T, dv, dk))
    I = np.zeros((T, dv, dk))
    for t in range(T):
        accM = np.zeros((dv, dk))
        accJ = np.zeros((dv, dk))
        for s in range(t + 1):
            w = 1.0
            for r in range(s + 1, t + 1):
                w *= f[r]
            accM += w * np.outer(v[s], k[s])
            accJ += w * np.outer(b[s], k[s] * k[s])
        w0 = 1.0
        for r in range(t + 1):
            w0 *= f[r]
        M[t] = accM + w0 * M0
        I[t] = accJ + w0 * J0 + float(Ip)
    return M, I


def direct_sum_outputs(q, k, v, b, gt, g, Ip, scale, mu0=None, I0=None):
    """o, o_var (kernel convention, scale**1) of one (sequence, head), float64."""
    M, I = direct_sum_states(k, v, b, gt, g, Ip, mu0, I0)
    q = np.asarray(q, np.float64)
    o = scale * np.einsum("tdn,tn->td", M / I, q)
    ov = scale * np.einsum("tdn,tn->td", 1.0 / I, q * q)
    return o, ov, M[-1] / I[-1], I[-1]


# --------------------------------------------------------------------------
# hand-derived backward (what the HIP kernels implement), one (sequence, head)
# --------------------------------------------------------------------------
def backward_formulas(q, k, v, b, gt, g, Ip, scale, do, dovar=None, mu0=None, I0=None):
    """Closed-form gradients of one (sequence, head) in float64 numpy.

    Mirrors the structure of the reference's backward kernel
    (chunk...py:360-430) with two deliberate differences that the tests pin
    against autograd: (i) d(log f) is obtained from the reverse cumulative sum
      dlogf_s = sum_{t>=s} ( <dMloc_t,M_t> + <dJloc_t,J_t> - <v_t,dv_t> - <b_t,db_t> )
    instead of dividing the state by f (chunk...py:409-412);
    (ii) with an initial state, dIp also receives -sum(dJ_0) and the
    initial-state gradients are returned (the reference returns None,
    chunk...py:617-620).

    Returns dict(dq, dk, dv, db, dgt, dg, dIp, dmu0, dI0).
    """
    q, k, v, b, gt, do = [np.asarray(x, np.float64) for x in (q, k, v, b, gt, do)]
    T, dk_ = k.shape
    dv_ = v.shape[1]
    g = float(g)
    Ip = float(Ip)
    f = np.exp(-gt * g)
    M, I = direct_sum_states(k, v, b, gt, g, Ip, mu0, I0)
    J = I - Ip
    has_var = dovar is not None
    if has_var:
        dovar = np.asarray(dovar, np.float64)
    dq = np.zeros_like(q)
    dkk = np.zeros_like(k)
    dvv = np.zeros_like(v)
    dbb = np.zeros_like(b)
    e = np.zeros(T)
    sigma = np.zeros(T)
    dM = np.zeros((dv_, dk_))
    dJ = np.zeros((dv_, dk_))
    for t in range(T - 1, -1, -1):
        G = scale * np.outer(do[t], q[t])
        rI = 1.0 / I[t]
        mu = M[t] * rI
        dMloc = G * rI
        dJloc = -dMloc * mu
        dq[t] = scale * (mu.T @ do[t])
        alpha = np.sum(dMloc * M[t])
        if has_var:
            dJloc = dJloc - scale * np.outer(dovar[t], q[t] * q[t]) * rI * rI
            dq[t] += 2.0 * scale * q[t] * (rI.T @ dovar[t])
        alpha += np.sum(dJloc * J[t])
        sigma[t] = dJloc.sum()
        f_next = f[t + 1] if t + 1 < T else 0.0
        dM = dMloc + f_next * dM
        dJ = dJloc + f_next * dJ
        dvv[t] = dM @ k[t]
        dbb[t] = dJ @ (k[t] * k[t])
        dkk[t] = dM.T @ v[t] + 2.0 * k[t] * (dJ.T @ b[t])
        e[t] = alpha - v[t] @ dvv[t] - b[t] @ dbb[t]
    dlogf = np.cumsum(e[::-1])[::-1]
    dgt = -g * dlogf
    dg = -(gt * dlogf).sum()
    # carries that flow into the initial state (M_0, J_0)
    dM0 = f[0] * dM
    dJ0 = f[0] * dJ
    dIp = sigma.sum()
    out = dict(dq=dq, dk=dkk, dv=dvv, db=dbb, dgt=dgt, dg=dg)
    if mu0 is not None:
        mu0 = np.asarray(mu0, np.float64)
        I0 = np.asarray(I0, np.float64)
        # M_0 = mu0*I0, J_0 = I0 - Ip
        out["dmu0"] = dM0 * I0
        out["dI0"] = dM0 * mu0 + dJ0
        dIp = dIp - dJ0.sum()
    out["dIp"] = dIp
    return out


# --------------------------------------------------------------------------
# integer helpers for varlen chunking
# --------------------------------------------------------------------------
def chunk_offsets(cu_seqlens: Sequence[int], chunk_size: int):
    """Cumulative per-document chunk counts, length N+1 (call site chunk...py:633)."""
    out = [0]
    for n in range(len(cu_seqlens) - 1):
        ln = int(cu_seqlens[n + 1]) - int(cu_seqlens[n])
        out.append(out[-1] + (ln + chunk_size - 1) // chunk_size)
    return out


def build_chunk_table(cu_seqlens: Sequence[int], chunk_size: int):
    """List of (doc, first_token, n_tokens) per chunk; chunks never straddle documents."""
    rows = []
    for n in range(len(cu_seqlens) - 1):
        s, e = int(cu_seqlens[n]), int(cu_seqlens[n + 1])
        for c0 in range(s, e, chunk_size):
            rows.append((n, c0, min(chunk_size, e - c0)))
    return rows


# --------------------------------------------------------------------------
# synthetic inputs of the benchmark configurations
# --------------------------------------------------------------------------
def make_inputs(B, T, H, dk, dv, seed=0, dtype=torch.float32, g_value=1.0, normalize_qk=True):
    """Seeded inputs: q,k ~ N(0,1) then L2-normalised per head; v ~ N(0,1);
    gt = sigmoid(N(0,1)) [B,T,H]; b = sigmoid(N(0,1)) [B,T,H,dv]; g = g_value, Ip = 1.
    Generated on the CPU generator in fp32 and then cast, so that every machine
    with the same torch build sees the same values."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn(B, T, H, dk, generator=gen)
    k = torch.randn(B, T, H, dk, generator=gen)
    v = torch.randn(B, T, H, dv, generator=gen)
    b = torch.sigmoid(torch.randn(B, T, H, dv, generator=gen))
    gt = torch.sigmoid(torch.randn(B, T, H, generator=gen))
    if normalize_qk:
        q = torch.nn.functional.normalize(q, p=2, dim=-1)
        k = torch.nn.functional.normalize(k, p=2, dim=-1)
    g = torch.full((H,), float(g_value))
    Ip = torch.ones(H)
    return dict(q=q.to(dtype), k=k.to(dtype), v=v.to(dtype), b=b.to(dtype), gt=gt, g=g, Ip=Ip)


def make_varlen_lengths(total_tokens=32768, mu=6.5, sigma=1.0, lo=16, hi=4096, seed=0):
    """Document lengths ~ round(exp(N(mu,sigma))) clipped to [lo,hi], drawn until the
    sum reaches ``total_tokens``; the last one is truncated to fit (merged into the
    previous one when it would be shorter than ``lo``)."""
    rng = np.random.RandomState(seed)
    lens = []
    tot = 0
    while tot < total_tokens:
        ln = int(np.clip(round(math.exp(rng.normal(mu, sigma))), lo, hi))
        ln = min(ln, total_tokens - tot)
        if ln < lo and lens:
            lens[-1] += ln
        else:
            lens.append(ln)
        tot += ln
    cu = [0]
    for ln in lens:
        cu.append(cu[-1] + ln)
    return cu
