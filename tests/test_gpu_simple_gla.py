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


@pytest.mark.parametrize("B,T,H,dk,dv,dtype", [
    (2, 64, 2, 64, 64, torch.bfloat16),      # exactly one tile
    (1, 1, 1, 16, 16, torch.bfloat16),       # one token, smallest head dims
    (2, 333, 3, 48, 80, torch.bfloat16),     # key dim not a multiple of 32, ragged last tile
    (1, 257, 2, 128, 128, torch.bfloat16),
    (1, 130, 1, 256, 256, torch.bfloat16),   # largest head dims
    (1, 100, 2, 40, 24, torch.bfloat16),     # head dims padded by the host to multiples of 16
    (2, 150, 2, 64, 32, torch.float32),      # fp32 rows (operands are rounded to bf16 in the kernel)
])
def test_forward_only_kernel_shapes(gpu_device, B, T, H, dk, dv, dtype):
    """The forward of its own that chunk_simple_gla takes without autograd, against the closed form and against
    the autograd path (the Palimpsa kernels on b = 0) on the same inputs."""
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    q, k, v, g, S0 = _inputs(B, T, H, dk, dv, 21)
    q, k, v = (x.to(dtype) for x in (q, k, v))
    dev = gpu_device
    with torch.no_grad():
        o, S = chunk_simple_gla(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g.to(dev), scale=0.7,
                                initial_state=S0.to(dev), output_final_state=True)
    assert o.dtype == dtype and o.shape == (B, T, H, dv) and S.shape == (B, H, dk, dv)
    o_ref, S_ref = _closed_form(q, k, v, g, 0.7, S0)
    assert hp.max_abs(o.float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(S, S_ref) <= 1e-2
    if dk + 2 * dv > 600:
        return          # beyond the LDS budget of the Palimpsa tile-state kernel, which stages k, v and b in fp32
    qg = q.to(dev).requires_grad_(True)
    o_g, S_g = chunk_simple_gla(q=qg, k=k.to(dev), v=v.to(dev), g=g.to(dev), scale=0.7,
                                initial_state=S0.to(dev), output_final_state=True)
    assert o_g.grad_fn is not None
    assert hp.max_abs(o.float(), o_g.float()) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(S, S_g) <= 1e-2


def test_forward_only_strong_and_weak_decay(gpu_device):
    """Decay so strong that a tile forgets its start, and none at all (g = 0: plain causal linear attention)."""
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    B, T, H, dk, dv = 1, 192, 2, 64, 64
    q, k, v, g, S0 = _inputs(B, T, H, dk, dv, 22)
    g = torch.stack([torch.full((B, T), -3.0), torch.zeros(B, T)], dim=-1)
    dev = gpu_device
    with torch.no_grad():
        o, S = chunk_simple_gla(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g.to(dev), initial_state=S0.to(dev),
                                output_final_state=True)
    o_ref, S_ref = _closed_form(q, k, v, g, dk ** -0.5, S0)
    assert hp.max_abs(o.float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(S, S_ref) <= 1e-2


def test_forward_only_full_size_against_token_serial(gpu_device):
    """Headline shape (B=8, T=2048, H=12, d=64): whole result against the token-serial fp32-state kernel, a slice
    against the closed form."""
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla, fused_recurrent_simple_gla
    B, T, H, d = 8, 2048, 12, 64
    q, k, v, g, S0 = _inputs(B, T, H, d, d, 23)
    dev = gpu_device
    args = dict(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g.to(dev), initial_state=S0.to(dev), output_final_state=True)
    with torch.no_grad():
        o, S = chunk_simple_gla(**args)
        o_r, S_r = fused_recurrent_simple_gla(**args)
    assert hp.max_abs(o.float(), o_r.float()) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(S, S_r) <= 1e-2
    bs, hs = [5], [0, 11]
    sub = lambda x: x[bs][:, :512][:, :, hs]
    o_ref, _ = _closed_form(sub(q), sub(k), sub(v), sub(g), d ** -0.5, S0[bs][:, hs])
    assert hp.max_abs(o[bs][:, :512][:, :, hs].float(), o_ref) <= hp.BF16_OUT_ABS_TOL


def test_forward_only_rejects_bad_arguments(gpu_device):
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    q, k, v, g, _ = _inputs(2, 70, 2, 32, 32, 24)
    dev = gpu_device
    with pytest.raises(ValueError):
        chunk_simple_gla(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=None)
    with pytest.raises(ValueError):
        chunk_simple_gla(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g.to(dev), cu_seqlens=torch.tensor([0, 70], device=dev))
    with pytest.raises(ValueError):
        chunk_simple_gla(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g[:, :10].to(dev))
