"""Scalar-gated linear attention through the Palimpsa kernels (b = 0, Ip = 1) against the closed form

    o = scale * ((Q K^T) * L) V + scale * F * (Q S_0),   L[t,s] = exp(c_t - c_s) for s <= t,  c = cumsum(g)

evaluated in float64 as dense masked matmuls (independent of the recurrence oracle), forward and, by
autograd through the closed form, backward.  Bars as for the other bf16-input kernels.
"""
import pytest
import torch

from tests import helpers as hp

pytestmark = pytest.mark.gpu


def _closed_form(q, k, v, g, scale, S0=None):
    """float64, [B,T,H,*]; returns o [B,T,H,dv], S_T [B,H,dk,dv]."""
    q, k, v, g = (x.double() for x in (q, k, v, g))
    c = g.cumsum(1)                                               # [B,T,H]
    L = torch.exp(c[:, :, None] - c[:, None, :])                  # [B,t,s,H]
    T = q.shape[1]
    mask = torch.tril(torch.ones(T, T, dtype=torch.bool))[None, :, :, None]
    L = torch.where(mask, L, torch.zeros_like(L))
    A = torch.einsum("bthn,bshn->btsh", q, k) * L
    o = torch.einsum("btsh,bshd->bthd", A, v)
    a_end = torch.exp(c[:, -1:, :] - c)                           # decay from s to the end
    S = torch.einsum("bshn,bsh,bshd->bhnd", k, a_end, v)
    if S0 is not None:
        S0 = S0.double()
        o = o + torch.einsum("bthn,bhnd->bthd", q * torch.exp(c)[..., None], S0)
        S = S + torch.exp(c[:, -1])[..., None, None] * S0
    return o * scale, S


def _inputs(B, T, H, dk, dv, seed):
    gen = torch.Generator().manual_seed(seed)
    q = torch.nn.functional.normalize(torch.randn(B, T, H, dk, generator=gen), dim=-1).bfloat16()
    k = torch.nn.functional.normalize(torch.randn(B, T, H, dk, generator=gen), dim=-1).bfloat16()
    v = torch.randn(B, T, H, dv, generator=gen).bfloat16()
    g = -torch.nn.functional.softplus(torch.randn(B, T, H, generator=gen)) * torch.linspace(0.05, 2.0, H)
    S0 = torch.randn(B, H, dk, dv, generator=gen) * 0.2
    return q, k, v, g, S0


@pytest.mark.parametrize("which", ["chunk", "recurrent"])
def test_forward_and_state_against_closed_form(gpu_device, which):
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla, fused_recurrent_simple_gla
    op = chunk_simple_gla if which == "chunk" else fused_recurrent_simple_gla
    B, T, H, dk, dv = 2, 200, 3, 64, 32
    q, k, v, g, S0 = _inputs(B, T, H, dk, dv, 11)
    dev = gpu_device
    o, S = op(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g.to(dev), initial_state=S0.to(dev), output_final_state=True)
    o_ref, S_ref = _closed_form(q, k, v, g, dk ** -0.5, S0)
    assert S.shape == (B, H, dk, dv)
    assert hp.max_abs(o.float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(S, S_ref) <= 1e-2
    o2, none = op(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g.to(dev))
    assert none is None
    assert hp.max_abs(o2.float(), _closed_form(q, k, v, g, dk ** -0.5)[0]) <= hp.BF16_OUT_ABS_TOL


def test_chunk_backward_against_closed_form(gpu_device):
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    B, T, H, dk, dv = 1, 150, 2, 32, 64
    q, k, v, g, S0 = _inputs(B, T, H, dk, dv, 12)
    gen = torch.Generator().manual_seed(13)
    do = torch.randn(B, T, H, dv, generator=gen)
    dev = gpu_device
    leaves = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g, S0)]
    o, _ = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], initial_state=leaves[4], scale=0.3)
    (o.float() * do.to(dev)).sum().backward()
    ref_leaves = [x.double().clone().requires_grad_(True) for x in (q, k, v, g, S0)]
    o_ref, _ = _closed_form(*ref_leaves[:4], 0.3, ref_leaves[4])
    (o_ref * do.double()).sum().backward()
    for name, x, r in zip(("q", "k", "v", "g", "S0"), leaves, ref_leaves):
        err = hp.max_rel(x.grad, r.grad)
        assert err <= hp.BF16_GRAD_NORM_TOL, (name, err)


def test_packed_documents(gpu_device):
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    H, dk, dv = 2, 32, 32
    cu = [0, 70, 71, 200]
    q, k, v, g, _ = _inputs(1, cu[-1], H, dk, dv, 14)
    dev = gpu_device
    o, S = chunk_simple_gla(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g.to(dev), output_final_state=True,
                            cu_seqlens=torch.tensor(cu, device=dev))
    for j in range(len(cu) - 1):
        sl = slice(cu[j], cu[j + 1])
        o_ref, S_ref = _closed_form(q[:, sl], k[:, sl], v[:, sl], g[:, sl], dk ** -0.5)
        assert hp.max_abs(o[:, sl].float(), o_ref) <= hp.BF16_OUT_ABS_TOL
        assert hp.max_rel(S[j:j + 1], S_ref) <= 1e-2
