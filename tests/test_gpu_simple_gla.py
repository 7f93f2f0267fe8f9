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
    """pal_gla_chunk_fwd against the closed form and against the Palimpsa kernels on b = 0, Ip = 1."""
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
    # second implementation: the Palimpsa kernels on b = 0, Ip = 1
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa
    ones = torch.ones(H, device=dev)
    with torch.no_grad():
        o_p, mu_p, _ = chunk_palimpsa(q.to(dev), k.to(dev), v.to(dev), torch.zeros_like(v).to(dev), -g.to(dev), ones, ones,
                                      scale=0.7, initial_mu_state=S0.transpose(-1, -2).contiguous().to(dev),
                                      initial_I_state=torch.ones(B, H, dv, dk, device=dev), output_final_state=True)
    assert hp.max_abs(o.float(), o_p.float()) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(S, mu_p.transpose(-1, -2)) <= 1e-2


@pytest.mark.parametrize("B,T,H,dk,dv,dtype", [
    (2, 64, 2, 64, 64, torch.bfloat16),
    (1, 1, 1, 16, 16, torch.bfloat16),
    (2, 333, 3, 48, 80, torch.bfloat16),
    (1, 257, 2, 128, 128, torch.bfloat16),
    (1, 130, 1, 256, 256, torch.bfloat16),
    (1, 100, 2, 40, 24, torch.bfloat16),
    (2, 150, 2, 64, 32, torch.float32),
])
def test_backward_shapes_against_closed_form(gpu_device, B, T, H, dk, dv, dtype):
    """Gradients of q, k, v, g and the initial state from pal_gla_chunk_bwd against autograd through the dense
    float64 closed form; normalised by the largest reference entry, bar as for the other bf16-input kernels."""
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    q, k, v, g, S0 = _inputs(B, T, H, dk, dv, 31)
    q, k, v = (x.to(dtype) for x in (q, k, v))
    gen = torch.Generator().manual_seed(32)
    do = torch.randn(B, T, H, dv, generator=gen)
    dev = gpu_device
    leaves = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g, S0)]
    o, _ = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], initial_state=leaves[4], scale=0.5)
    (o.float() * do.to(dev)).sum().backward()
    ref_leaves = [x.double().clone().requires_grad_(True) for x in (q, k, v, g, S0)]
    o_ref, _ = _closed_form(*ref_leaves[:4], 0.5, ref_leaves[4])
    (o_ref * do.double()).sum().backward()
    assert hp.max_abs(o.float(), o_ref.detach()) <= hp.BF16_OUT_ABS_TOL
    for name, x, r in zip(("q", "k", "v", "g", "S0"), leaves, ref_leaves):
        assert x.grad.shape == r.grad.shape and x.grad.dtype == x.dtype
        err = hp.max_rel(x.grad, r.grad)
        assert err <= hp.BF16_GRAD_NORM_TOL, (name, err)


def test_backward_packed_documents(gpu_device):
    """Every document of a packed batch gets the gradients of a run of its own (gate gradients do not leak
    across document boundaries)."""
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    H, dk, dv = 2, 32, 64
    cu = [0, 70, 71, 200, 264]
    q, k, v, g, _ = _inputs(1, cu[-1], H, dk, dv, 33)
    gen = torch.Generator().manual_seed(34)
    do = torch.randn(1, cu[-1], H, dv, generator=gen)
    dev = gpu_device
    leaves = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g)]
    o, _ = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], cu_seqlens=torch.tensor(cu, device=dev))
    (o.float() * do.to(dev)).sum().backward()
    for j in range(len(cu) - 1):
        sl = slice(cu[j], cu[j + 1])
        ref_leaves = [x[:, sl].double().clone().requires_grad_(True) for x in (q, k, v, g)]
        o_ref, _ = _closed_form(*ref_leaves, dk ** -0.5)
        (o_ref * do[:, sl].double()).sum().backward()
        for name, x, r in zip(("q", "k", "v", "g"), leaves, ref_leaves):
            err = hp.max_rel(x.grad[:, sl], r.grad)
            assert err <= hp.BF16_GRAD_NORM_TOL, (j, name, err)


def test_backward_full_size_against_palimpsa_kernels(gpu_device):
    """Headline shape: gradients against those of the Palimpsa kernels on b = 0, Ip = 1 (independent code), and
    the result is bitwise reproducible."""
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa
    B, T, H, d = 8, 2048, 12, 64
    q, k, v, g, _ = _inputs(B, T, H, d, d, 35)
    gen = torch.Generator().manual_seed(36)
    do = torch.randn(B, T, H, d, generator=gen).bfloat16()
    dev = gpu_device

    def run():
        leaves = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g)]
        o, _ = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3])
        o.backward(do.to(dev))
        return o, [x.grad for x in leaves]

    o, grads = run()
    o2, grads2 = run()
    assert torch.equal(o, o2) and all(torch.equal(a, b) for a, b in zip(grads, grads2))
    leaves = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g)]
    ones = torch.ones(H, device=dev)
    o_p = chunk_palimpsa(leaves[0], leaves[1], leaves[2], torch.zeros_like(leaves[2]), -leaves[3], ones, ones)
    o_p.backward(do.to(dev))
    assert hp.max_abs(o.float(), o_p.float()) <= hp.BF16_OUT_ABS_TOL
    for name, x, r in zip(("q", "k", "v", "g"), grads, leaves):
        err = hp.max_rel(x, r.grad)
        assert err <= hp.BF16_GRAD_NORM_TOL, (name, err)


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


@pytest.mark.parametrize("H,dk,dv", [(16, 48, 96), (16, 96, 192), (4, 96, 96)])
def test_reference_config_shapes(gpu_device, H, dk, dv):
    """Head shapes of the reference's configurations that run this path (mamba2_170M: state 48, head 96;
    mamba2_760M and not_palimpsa_760M: 96 / 192), scale = 1 as the Mamba2-style layer passes it: chunked forward
    and backward, token-serial forward."""
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla, fused_recurrent_simple_gla
    B, T = 1, 200
    q, k, v, g, S0 = _inputs(B, T, H, dk, dv, 41)
    gen = torch.Generator().manual_seed(42)
    do = torch.randn(B, T, H, dv, generator=gen)
    dev = gpu_device
    leaves = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g, S0)]
    o, S = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], initial_state=leaves[4], scale=1.0,
                            output_final_state=True)
    (o.float() * do.to(dev)).sum().backward()
    ref_leaves = [x.double().clone().requires_grad_(True) for x in (q, k, v, g, S0)]
    o_ref, S_ref = _closed_form(*ref_leaves[:4], 1.0, ref_leaves[4])
    (o_ref * do.double()).sum().backward()
    tol = hp.BF16_OUT_ABS_TOL * max(1.0, o_ref.abs().max().item())
    assert hp.max_abs(o.float(), o_ref.detach()) <= tol
    assert hp.max_rel(S, S_ref.detach()) <= 1e-2
    for name, x, r in zip(("q", "k", "v", "g", "S0"), leaves, ref_leaves):
        err = hp.max_rel(x.grad, r.grad)
        assert err <= hp.BF16_GRAD_NORM_TOL, (name, err)
    with torch.no_grad():
        o_r, S_r = fused_recurrent_simple_gla(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g.to(dev), scale=1.0,
                                              initial_state=S0.to(dev), output_final_state=True)
    assert hp.max_abs(o_r.float(), o_ref.detach()) <= tol
    assert hp.max_rel(S_r, S_ref.detach()) <= hp.FP32_REL_TOL


def test_decode_steps_in_place_and_packed(gpu_device):
    """Single-token calls with the state fed back equal one multi-token call; packed documents equal separate
    runs; fp32 rows meet the fp32 bar."""
    from palimpsa_amd.ops.simple_gla import fused_recurrent_simple_gla
    B, T, H, dk, dv = 3, 12, 2, 64, 80
    q, k, v, g, S0 = _inputs(B, T, H, dk, dv, 43)
    q, k, v = q.float(), k.float(), v.float()
    dev = gpu_device
    qd, kd, vd, gd = (x.to(dev) for x in (q, k, v, g))
    S = S0.to(dev)
    outs = []
    with torch.no_grad():
        for t in range(T):
            o, S = fused_recurrent_simple_gla(q=qd[:, t:t + 1], k=kd[:, t:t + 1], v=vd[:, t:t + 1], g=gd[:, t:t + 1],
                                              initial_state=S, output_final_state=True)
            outs.append(o)
        o_all, S_all = fused_recurrent_simple_gla(q=qd, k=kd, v=vd, g=gd, initial_state=S0.to(dev), output_final_state=True)
    o_steps = torch.cat(outs, dim=1)
    o_ref, S_ref = _closed_form(q, k, v, g, dk ** -0.5, S0)
    assert hp.max_rel(o_steps, o_ref) <= hp.FP32_REL_TOL and hp.max_rel(o_all, o_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(S, S_ref) <= hp.FP32_REL_TOL and hp.max_rel(S_all, S_ref) <= hp.FP32_REL_TOL
    # packed documents
    cu = [0, 5, 6, 20, 36]
    q2, k2, v2, g2, _ = _inputs(1, cu[-1], H, dk, dv, 44)
    with torch.no_grad():
        o2, S2 = fused_recurrent_simple_gla(q=q2.to(dev), k=k2.to(dev), v=v2.to(dev), g=g2.to(dev), output_final_state=True,
                                            cu_seqlens=torch.tensor(cu, device=dev))
    for j in range(len(cu) - 1):
        sl = slice(cu[j], cu[j + 1])
        o_r, S_r = _closed_form(q2[:, sl], k2[:, sl], v2[:, sl], g2[:, sl], dk ** -0.5)
        assert hp.max_abs(o2[:, sl].float(), o_r) <= hp.BF16_OUT_ABS_TOL
        assert hp.max_rel(S2[j:j + 1], S_r) <= hp.FP32_REL_TOL


def test_recurrent_with_autograd_still_differentiates(gpu_device):
    from palimpsa_amd.ops.simple_gla import fused_recurrent_simple_gla
    q, k, v, g, S0 = _inputs(1, 40, 2, 32, 32, 45)
    dev = gpu_device
    leaves = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g)]
    o, _ = fused_recurrent_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], scale=0.4)
    o.float().sum().backward()
    ref_leaves = [x.double().clone().requires_grad_(True) for x in (q, k, v, g)]
    _closed_form(*ref_leaves, 0.4)[0].sum().backward()
    for name, x, r in zip(("q", "k", "v", "g"), leaves, ref_leaves):
        assert hp.max_rel(x.grad, r.grad) <= hp.BF16_GRAD_NORM_TOL, name


def test_packed_batch_with_empty_documents(gpu_device):
    """Documents of length zero (repeated cu_seqlens entries) take no tile; their final state is the initial one
    and the gradients of the others are untouched."""
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla, fused_recurrent_simple_gla
    H, dk, dv = 2, 32, 32
    cu = [0, 0, 70, 70, 135, 135]
    q, k, v, g, _ = _inputs(1, cu[-1], H, dk, dv, 51)
    gen = torch.Generator().manual_seed(52)
    S0 = torch.randn(len(cu) - 1, H, dk, dv, generator=gen) * 0.2
    do = torch.randn(1, cu[-1], H, dv, generator=gen)
    dev = gpu_device
    cu_d = torch.tensor(cu, device=dev)
    leaves = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g, S0)]
    o, S = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], initial_state=leaves[4],
                            output_final_state=True, cu_seqlens=cu_d)
    (o.float() * do.to(dev)).sum().backward()
    with torch.no_grad():
        o_r, S_r = fused_recurrent_simple_gla(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g.to(dev), initial_state=S0.to(dev),
                                              output_final_state=True, cu_seqlens=cu_d)
    for j in range(len(cu) - 1):
        sl = slice(cu[j], cu[j + 1])
        if cu[j + 1] == cu[j]:
            assert torch.equal(S[j].cpu(), S0[j]) and torch.equal(S_r[j].cpu(), S0[j])
            assert torch.equal(leaves[4].grad[j].cpu(), torch.zeros(H, dk, dv))
            continue
        ref_leaves = [x[:, sl].double().clone().requires_grad_(True) for x in (q, k, v, g)]
        S0_ref = S0[j:j + 1].double().clone().requires_grad_(True)
        o_ref, S_ref = _closed_form(*ref_leaves, dk ** -0.5, S0_ref)
        (o_ref * do[:, sl].double()).sum().backward()
        assert hp.max_abs(o[:, sl].float(), o_ref.detach()) <= hp.BF16_OUT_ABS_TOL
        assert hp.max_abs(o_r[:, sl].float(), o_ref.detach()) <= hp.BF16_OUT_ABS_TOL
        assert hp.max_rel(S[j:j + 1], S_ref.detach()) <= 1e-2 and hp.max_rel(S_r[j:j + 1], S_ref.detach()) <= hp.FP32_REL_TOL
        for name, x, r in zip(("q", "k", "v", "g"), leaves, ref_leaves):
            assert hp.max_rel(x.grad[:, sl], r.grad) <= hp.BF16_GRAD_NORM_TOL, (j, name)
        assert hp.max_rel(leaves[4].grad[j:j + 1], S0_ref.grad) <= hp.BF16_GRAD_NORM_TOL


def test_sequence_longer_than_one_scan_window(gpu_device):
    """More than 1024 tiles in one sequence: the state scans (forward and reverse) and the gate suffix sums work in
    windows.  Forward against the token-serial kernel, gradients against the Palimpsa kernels on b = 0, Ip = 1
    (both independent code), bf16 gates."""
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla, fused_recurrent_simple_gla
    B, T, H, dk, dv = 1, 1031 * 64 + 7, 2, 16, 32
    q, k, v, g, S0 = _inputs(B, T, H, dk, dv, 61)
    g = (g * 0.2).bfloat16()
    gen = torch.Generator().manual_seed(62)
    do = torch.randn(B, T, H, dv, generator=gen).bfloat16()
    dev = gpu_device
    leaves = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g, S0)]
    o, S = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], initial_state=leaves[4],
                            output_final_state=True)
    o.backward(do.to(dev))
    with torch.no_grad():
        o_r, S_r = fused_recurrent_simple_gla(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g.to(dev), initial_state=S0.to(dev),
                                              output_final_state=True)
    assert hp.max_abs(o.float(), o_r.float()) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(S, S_r) <= 1e-2
    ref = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g)]
    mu0 = S0.transpose(-1, -2).contiguous().to(dev).requires_grad_(True)
    ones = torch.ones(H, device=dev)
    o_p = chunk_palimpsa(ref[0], ref[1], ref[2], torch.zeros_like(ref[2]), -ref[3].float(), ones, ones,
                         initial_mu_state=mu0, initial_I_state=torch.ones_like(mu0))
    o_p.backward(do.to(dev))
    assert leaves[3].grad.dtype == torch.bfloat16
    for name, x, r in zip(("q", "k", "v"), leaves, ref):
        assert hp.max_rel(x.grad, r.grad) <= hp.BF16_GRAD_NORM_TOL, name
    # the gate gradient accumulates over up to 66 k tokens; bf16 output, compared where the reference is large
    assert hp.max_rel(leaves[3].grad.float(), ref[3].grad.float()) <= 2 * hp.BF16_GRAD_NORM_TOL
    assert hp.max_rel(leaves[4].grad, mu0.grad.transpose(-1, -2)) <= hp.BF16_GRAD_NORM_TOL


def test_random_shape_sweep(gpu_device):
    """Seeded random shapes (head dims any multiple of 8 up to 256 through the host-side padding, ragged lengths,
    packed or batched, with or without an initial state): forward and backward against the closed form."""
    import random
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    rng = random.Random(1234)
    dev = gpu_device
    for case in range(14):
        H = rng.choice([1, 2, 3, 5])
        dk = 8 * rng.randint(1, 32)
        dv = 8 * rng.randint(1, 32)
        packed = rng.random() < 0.4
        if packed:
            lens = [rng.randint(1, 150) for _ in range(rng.randint(1, 4))]
            B, T = 1, sum(lens)
            cu = [0]
            for ln in lens:
                cu.append(cu[-1] + ln)
        else:
            B, T, cu = rng.choice([1, 2]), rng.randint(1, 200), None
        with_state = rng.random() < 0.5
        scale = rng.choice([1.0, 0.37, dk ** -0.5])
        q, k, v, g, _ = _inputs(B, T, H, dk, dv, 1000 + case)
        n_seq = len(cu) - 1 if cu else B
        gen = torch.Generator().manual_seed(2000 + case)
        S0 = torch.randn(n_seq, H, dk, dv, generator=gen) * 0.2 if with_state else None
        do = torch.randn(B, T, H, dv, generator=gen)
        tensors = [q, k, v, g] + ([S0] if with_state else [])
        leaves = [x.to(dev).clone().requires_grad_(True) for x in tensors]
        o, S = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], scale=scale,
                                initial_state=leaves[4] if with_state else None, output_final_state=True,
                                cu_seqlens=torch.tensor(cu, device=dev) if cu else None)
        (o.float() * do.to(dev)).sum().backward()
        ref = [x.double().clone().requires_grad_(True) for x in tensors]
        if cu:
            outs, states = [], []
            for j in range(n_seq):
                sl = slice(cu[j], cu[j + 1])
                o_j, S_j = _closed_form(ref[0][:, sl], ref[1][:, sl], ref[2][:, sl], ref[3][:, sl], scale,
                                        ref[4][j:j + 1] if with_state else None)
                outs.append(o_j)
                states.append(S_j)
            o_ref, S_ref = torch.cat(outs, dim=1), torch.cat(states, dim=0)
        else:
            o_ref, S_ref = _closed_form(ref[0], ref[1], ref[2], ref[3], scale, ref[4] if with_state else None)
        (o_ref * do.double()).sum().backward()
        tag = (case, B, T, H, dk, dv, cu, with_state)
        assert hp.max_abs(o.float(), o_ref.detach()) <= hp.BF16_OUT_ABS_TOL * max(1.0, o_ref.abs().max().item()), tag
        assert hp.max_rel(S, S_ref.detach()) <= 1e-2, tag
        for name, x, r in zip(("q", "k", "v", "g", "S0"), leaves, ref):
            assert hp.max_rel(x.grad, r.grad) <= hp.BF16_GRAD_NORM_TOL, (name,) + tag


def test_prefill_then_decode(gpu_device):
    """Serving flow: chunked prefill returns the state in the cache's [N,H,dk,dv] layout, single-token decode steps
    continue from it; the outputs equal those of one pass over the whole sequence."""
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla, fused_recurrent_simple_gla
    B, T0, T1, H, dk, dv = 2, 150, 6, 2, 64, 96
    q, k, v, g, _ = _inputs(B, T0 + T1, H, dk, dv, 71)
    dev = gpu_device
    qd, kd, vd, gd = (x.to(dev) for x in (q, k, v, g))
    with torch.no_grad():
        o0, S = chunk_simple_gla(q=qd[:, :T0], k=kd[:, :T0], v=vd[:, :T0], g=gd[:, :T0], output_final_state=True)
        outs = [o0]
        for t in range(T0, T0 + T1):
            o, S = fused_recurrent_simple_gla(q=qd[:, t:t + 1], k=kd[:, t:t + 1], v=vd[:, t:t + 1], g=gd[:, t:t + 1],
                                              initial_state=S, output_final_state=True)
            outs.append(o)
    o_all = torch.cat(outs, dim=1)
    o_ref, S_ref = _closed_form(q, k, v, g, dk ** -0.5)
    assert hp.max_abs(o_all.float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(S, S_ref) <= 1e-2


def test_bound_decode_step_and_graph_replay(gpu_device):
    """SimpleGlaDecodeStep: same kernel as fused_recurrent_simple_gla, so results agree exactly; recorded into a HIP
    graph, every replay (with eager work in between) agrees with the eager result too."""
    from palimpsa_amd.ops.simple_gla import SimpleGlaDecodeStep, fused_recurrent_simple_gla
    B, H, dk, dv, steps = 5, 3, 64, 48, 6
    q, k, v, g, S0 = _inputs(B, steps, H, dk, dv, 81)
    dev = gpu_device
    qd, kd, vd, gd = (x.to(dev) for x in (q, k, v, g))
    S = S0.to(dev)
    outs = []
    with torch.no_grad():
        for t in range(steps):
            o, S = fused_recurrent_simple_gla(q=qd[:, t:t + 1], k=kd[:, t:t + 1], v=vd[:, t:t + 1], g=gd[:, t:t + 1],
                                              initial_state=S, output_final_state=True)
            outs.append(o)
    dec = SimpleGlaDecodeStep(B, H, dk, dv, dev)
    buf = [torch.empty_like(x[:, :1].contiguous()) for x in (qd, kd, vd, gd)]
    Sb = S0.to(dev).clone()
    dec.bind(buf[0], buf[1], buf[2], buf[3], Sb)
    for t in range(steps):
        for b_, x in zip(buf, (qd, kd, vd, gd)):
            b_.copy_(x[:, t:t + 1])
        assert torch.equal(dec.step(), outs[t])
    assert torch.equal(Sb, S)
    # graph
    Sb.copy_(S0.to(dev))
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        dec.step()
        Sb.copy_(S0.to(dev))
        with torch.cuda.graph(graph, stream=side):
            dec.step()
    torch.cuda.current_stream().wait_stream(side)
    for t in range(steps):
        for b_, x in zip(buf, (qd, kd, vd, gd)):
            b_.copy_(x[:, t:t + 1])
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(dec.o, outs[t]), t
    assert torch.equal(Sb, S)
    # blocks of three tokens against the closed form
    dec3 = SimpleGlaDecodeStep(B, H, dk, dv, dev, tokens=3)
    buf3 = [torch.empty_like(x[:, :3].contiguous()) for x in (qd, kd, vd, gd)]
    S3 = S0.to(dev).clone()
    dec3.bind(buf3[0], buf3[1], buf3[2], buf3[3], S3)
    o3 = []
    for t in range(0, steps, 3):
        for b_, x in zip(buf3, (qd, kd, vd, gd)):
            b_.copy_(x[:, t:t + 3])
        o3.append(dec3.step().clone())
    o_ref, S_ref = _closed_form(q, k, v, g, dk ** -0.5, S0)
    assert hp.max_abs(torch.cat(o3, dim=1).float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(S3, S_ref) <= hp.FP32_REL_TOL
    with pytest.raises(ValueError):
        dec.bind(buf[0].float(), buf[1], buf[2], buf[3], Sb)
    with pytest.raises(ValueError):
        SimpleGlaDecodeStep(B, H, 40, dv, dev)


def test_packed_pretraining_batch_full_size(gpu_device):
    """The packed-batch benchmark shape (32768 tokens in 23 documents, H=16, d=96) on the path without the precision
    state: forward against the token-serial kernel, gradients against the Palimpsa kernels on b = 0, Ip = 1."""
    from oracle import palimpsa_oracle as po
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla, fused_recurrent_simple_gla
    cu = po.make_varlen_lengths(32768, seed=0)
    T, H, d = cu[-1], 16, 96
    q, k, v, g, _ = _inputs(1, T, H, d, d, 91)
    gen = torch.Generator().manual_seed(92)
    do = torch.randn(1, T, H, d, generator=gen).bfloat16()
    dev = gpu_device
    cu_d = torch.tensor(cu, device=dev, dtype=torch.int32)
    leaves = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g)]
    o, S = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], output_final_state=True, cu_seqlens=cu_d)
    o.backward(do.to(dev))
    with torch.no_grad():
        o_r, S_r = fused_recurrent_simple_gla(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g.to(dev), output_final_state=True,
                                              cu_seqlens=cu_d)
    assert hp.max_abs(o.float(), o_r.float()) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(S, S_r) <= 1e-2
    ref = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g)]
    ones = torch.ones(H, device=dev)
    o_p = chunk_palimpsa(ref[0], ref[1], ref[2], torch.zeros_like(ref[2]), -ref[3], ones, ones, cu_seqlens=cu_d)
    o_p.backward(do.to(dev))
    for name, x, r in zip(("q", "k", "v", "g"), leaves, ref):
        assert hp.max_rel(x.grad, r.grad) <= hp.BF16_GRAD_NORM_TOL, name


def test_backward_packed_batch_walked_by_resident_workgroups(gpu_device):
    """Head dims up to 64 take the kernel that forms dq, dk, dv from one copy of the rows; its workgroups walk over
    several (tile, head) items each and request the tile table two items ahead.  8192 tokens in ragged documents
    (tiles of 1 to 64 tokens, 2000 items): gradients against the Palimpsa kernels on b = 0, Ip = 1 and, for three
    documents, against the closed form."""
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    H, dk, dv = 12, 64, 48
    lens, tot, j = [], 0, 0
    while tot < 8192:
        ln = min(1 + (j * 977) % 700, 8192 - tot)
        lens.append(ln)
        tot += ln
        j += 1
    cu = [0]
    for ln in lens:
        cu.append(cu[-1] + ln)
    q, k, v, g, _ = _inputs(1, cu[-1], H, dk, dv, 95)
    gen = torch.Generator().manual_seed(96)
    do = torch.randn(1, cu[-1], H, dv, generator=gen).bfloat16()
    dev = gpu_device
    cu_d = torch.tensor(cu, device=dev, dtype=torch.int32)
    leaves = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g)]
    o, _ = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], cu_seqlens=cu_d)
    o.backward(do.to(dev))
    ref = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g)]
    ones = torch.ones(H, device=dev)
    o_p = chunk_palimpsa(ref[0], ref[1], ref[2], torch.zeros_like(ref[2]), -ref[3], ones, ones, cu_seqlens=cu_d)
    o_p.backward(do.to(dev))
    for name, x, r in zip(("q", "k", "v", "g"), leaves, ref):
        assert hp.max_rel(x.grad, r.grad) <= hp.BF16_GRAD_NORM_TOL, name
    for jdoc in (0, len(lens) // 2, len(lens) - 1):
        sl = slice(cu[jdoc], cu[jdoc + 1])
        rl = [x[:, sl].double().clone().requires_grad_(True) for x in (q, k, v, g)]
        o_ref, _ = _closed_form(*rl, dk ** -0.5)
        (o_ref * do[:, sl].double()).sum().backward()
        for name, x, r in zip(("q", "k", "v", "g"), leaves, rl):
            assert hp.max_rel(x.grad[:, sl], r.grad) <= hp.BF16_GRAD_NORM_TOL, (jdoc, name)


def test_forward_and_backward_replay_in_a_graph(gpu_device):
    """chunk_simple_gla forward + backward recorded into a HIP graph (head dims 64: the backward tile kernel with
    resident workgroups): three replays on new values, with eager work in between, each equal to the eager result."""
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    dev = gpu_device
    B, T, H, d = 2, 300, 3, 64

    def fresh(seed):
        q, k, v, g, _ = _inputs(B, T, H, d, d, seed)
        do = torch.randn(B, T, H, d, generator=torch.Generator().manual_seed(seed + 1)).bfloat16()
        return [x.to(dev) for x in (q, k, v, g)], do.to(dev)

    def eager(xs, do):
        leaves = [x.clone().requires_grad_(True) for x in xs]
        o, _ = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3])
        return (o.detach(),) + torch.autograd.grad(o, leaves, do)

    xs0, do0 = fresh(500)
    static = [x.clone().requires_grad_(True) for x in xs0]
    static_do = do0.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            o, _ = chunk_simple_gla(q=static[0], k=static[1], v=static[2], g=static[3])
            torch.autograd.grad(o, static, static_do)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        o_g, _ = chunk_simple_gla(q=static[0], k=static[1], v=static[2], g=static[3])
        grads_g = torch.autograd.grad(o_g, static, static_do)
    for seed in (510, 520, 530):
        xs, do = fresh(seed)
        ref = eager(xs, do)
        with torch.no_grad():
            for x, y in zip(static, xs):
                x.copy_(y)
            static_do.copy_(do)
        graph.replay()
        torch.cuda.synchronize()
        for a_, b_, n in zip((o_g,) + tuple(grads_g), ref, "oqkvg"):
            assert torch.equal(a_, b_), (seed, n)


@pytest.mark.parametrize("dk,dv,dtype", [(64, 64, torch.bfloat16), (48, 96, torch.bfloat16), (32, 64, torch.float32)])
def test_shared_qk_heads_are_indexed_not_repeated(gpu_device, dk, dv, dtype):
    """The MetaMamba2 layer with its precision state off repeats its B, C groups over the heads of a group before it
    calls simple-GLA (layers/meta_mamba2.py:281-282, then :319-323).  The entry points also take the un-repeated
    [B,T,Hq,dk] rows and index the shared ones: outputs, final state and every gradient must equal the dense closed
    form on the repeated rows, with dq, dk summed over the heads of each group.  64 x 64 bf16 runs the backward
    kernel that forms the three input gradients together, the other shapes the three launches; packed documents
    in the first case; the decode kernel on the same rows."""
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla, fused_recurrent_simple_gla
    B, T, H, G = 2, 200, 6, 2
    rep = H // G
    q, k, v, g, S0 = _inputs(B, T, H, dk, dv, 91)
    q = q[:, :, ::rep].repeat_interleave(rep, dim=2).contiguous()     # heads of a group carry the same rows
    k = k[:, :, ::rep].repeat_interleave(rep, dim=2).contiguous()
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    gen = torch.Generator().manual_seed(92)
    do = torch.randn(B, T, H, dv, generator=gen)
    ref_leaves = [x.double().clone().requires_grad_(True) for x in (q, k, v, g, S0)]
    o_ref, S_ref = _closed_form(*ref_leaves[:4], dk ** -0.5, ref_leaves[4])
    (o_ref * do.double()).sum().backward()
    ref = {n: x.grad for n, x in zip(("q", "k", "v", "g", "S0"), ref_leaves)}
    for n in ("q", "k"):
        ref[n] = ref[n].reshape(B, T, G, rep, dk).sum(3)
    dev = gpu_device
    leaves = dict(q=q[:, :, ::rep].contiguous(), k=k[:, :, ::rep].contiguous(), v=v, g=g, S0=S0)
    leaves = {n: x.to(dev).clone().requires_grad_(True) for n, x in leaves.items()}
    assert leaves["q"].shape == (B, T, G, dk)
    o, S = chunk_simple_gla(q=leaves["q"], k=leaves["k"], v=leaves["v"], g=leaves["g"], initial_state=leaves["S0"],
                            output_final_state=True)
    (o.float() * do.to(dev)).sum().backward()
    out_tol = hp.BF16_OUT_ABS_TOL
    assert hp.max_abs(o.float(), o_ref) <= out_tol
    assert hp.max_rel(S, S_ref) <= 1e-2
    for n, x in leaves.items():
        assert x.grad.shape == x.shape
        err = hp.max_rel(x.grad, ref[n])
        assert err <= hp.BF16_GRAD_NORM_TOL, (n, err)
    with torch.no_grad():
        o_r, S_r = fused_recurrent_simple_gla(q=leaves["q"], k=leaves["k"], v=leaves["v"], g=leaves["g"],
                                              initial_state=leaves["S0"], output_final_state=True)
    assert hp.max_abs(o_r.float(), o_ref) <= out_tol
    assert hp.max_rel(S_r, S_ref) <= (1e-2 if dtype == torch.bfloat16 else 1e-4)
    if dk == 64:
        # the same tokens as one packed row of three documents, no initial state: equal to the dense batch document
        # by document
        cu = torch.tensor([0, 130, 131, B * T], device=dev)
        pk = {n: leaves[n].detach().reshape(1, B * T, *leaves[n].shape[2:]).clone().requires_grad_(True) for n in ("q", "k", "v", "g")}
        o_p, _ = chunk_simple_gla(q=pk["q"], k=pk["k"], v=pk["v"], g=pk["g"], cu_seqlens=cu)
        (o_p.float() * do.to(dev).reshape(1, B * T, H, dv)).sum().backward()
        flat = lambda x: x.reshape(1, B * T, *x.shape[2:])
        o_parts = []
        for a, b_ in ((0, 130), (130, 131), (131, B * T)):
            lv = [flat(x)[:, a:b_].double().clone().requires_grad_(True) for x in (q, k, v, g)]
            o_d, _ = _closed_form(*lv, dk ** -0.5)
            (o_d * flat(do)[:, a:b_].double()).sum().backward()
            o_parts.append(o_d.detach())
            for n, x in zip(("q", "k", "v", "g"), lv):
                want = x.grad.reshape(1, b_ - a, G, rep, dk).sum(3) if n in ("q", "k") else x.grad
                if b_ - a > 1:      # (the gradients of a one-token document are exact zeros or single products)
                    err = hp.max_rel(pk[n].grad[:, a:b_], want)
                    assert err <= hp.BF16_GRAD_NORM_TOL, (n, a, err)
        assert hp.max_abs(o_p.float(), torch.cat(o_parts, dim=1)) <= out_tol
