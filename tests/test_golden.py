"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the oracle).

CPU part: the oracle and the seeded input generator still reproduce the stored vectors.
GPU part: the HIP paths hit the same stored vectors through the C ABI.
"""
import os

import numpy as np
import pytest
import torch

from oracle import palimpsa_oracle as po
from tests import helpers as hp
from tests.golden import make_golden as mg

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    return dict(np.load(os.path.join(GOLD, name), allow_pickle=False))


# ------------------------------------------------------------------ CPU: oracle vs fixtures
def test_oracle_reproduces_c0_fixture():
    ref, now = _load("c0_recurrent_fp32.npz"), mg.c0_case()
    assert np.array_equal(ref["q_head"], now["q_head"]) and np.array_equal(ref["gt_head"], now["gt_head"])
    for k in ("o_every16", "final_mu", "final_I"):
        assert np.allclose(ref[k], now[k], rtol=1e-5, atol=1e-6), k


def test_oracle_reproduces_grad_fixture():
    ref, now = _load("small_grad_state_var.npz"), mg.grad_case()
    for k in ref:
        assert np.allclose(ref[k], now[k], rtol=1e-9, atol=1e-11), k


def test_oracle_reproduces_varlen_fixture():
    ref, now = _load("varlen_forward.npz"), mg.varlen_case()
    for k in ("o", "final_mu", "final_I"):
        assert np.allclose(ref[k], now[k], rtol=1e-5, atol=1e-6), k


# ------------------------------------------------------------------ GPU: kernels vs fixtures
@pytest.mark.gpu
def test_gpu_recurrent_hits_c0_fixture(gpu_device):
    from palimpsa_amd.ops.palimpsa import fused_recurrent_palimpsa

    ref = _load("c0_recurrent_fp32.npz")
    d = hp.to_device(po.make_inputs(2, 256, 4, 32, 32, seed=0), gpu_device)
    o, mu, I = fused_recurrent_palimpsa(d["q"], d["k"], d["v"], d["b"], d["gt"], d["g"], d["Ip"],
                                        output_final_state=True)
    assert hp.max_rel(o[:, ::16], torch.from_numpy(ref["o_every16"])) <= hp.FP32_REL_TOL
    assert hp.max_rel(mu, torch.from_numpy(ref["final_mu"])) <= hp.FP32_REL_TOL
    assert hp.max_rel(I, torch.from_numpy(ref["final_I"])) <= hp.FP32_REL_TOL


@pytest.mark.gpu
def test_gpu_chunk_hits_grad_fixture(gpu_device):
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa

    ref = _load("small_grad_state_var.npz")
    B, T, H, dk, dv = 1, 70, 2, 16, 16
    inp = po.make_inputs(B, T, H, dk, dv, seed=5, dtype=torch.bfloat16)
    gen = torch.Generator().manual_seed(6)
    mu0 = torch.randn(B, H, dv, dk, generator=gen) * 0.1
    I0 = 1.0 + torch.rand(B, H, dv, dk, generator=gen)
    do = torch.randn(B, T, H, dv, generator=gen)
    dov = torch.randn(B, T, H, dv, generator=gen) * 0.3
    names = ["q", "k", "v", "b", "gt", "g", "Ip"]
    leaves = [inp[n].to(gpu_device).requires_grad_(True) for n in names]
    st = [mu0.to(gpu_device).requires_grad_(True), I0.to(gpu_device).requires_grad_(True)]
    (o, ov), fmu, fI = chunk_palimpsa(*leaves, initial_mu_state=st[0], initial_I_state=st[1], scale=0.5,
                                      chunk_size=64, output_final_state=True, output_uncertainty=True)
    ((o.float() * do.to(gpu_device)).sum() + (ov.float() * dov.to(gpu_device)).sum()).backward()
    assert hp.max_abs(o, torch.from_numpy(ref["o"])) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_abs(ov, torch.from_numpy(ref["o_var"])) <= hp.BF16_OUT_ABS_TOL
    for n, x in zip(names[:5] + ["Ip", "mu0", "I0"], leaves[:5] + [leaves[6]] + st):
        assert hp.max_rel(x.grad, torch.from_numpy(ref["d" + n])) <= hp.BF16_GRAD_NORM_TOL, n


@pytest.mark.gpu
def test_gpu_paths_hit_varlen_fixture(gpu_device):
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa, fused_recurrent_palimpsa

    ref = _load("varlen_forward.npz")
    d = hp.to_device(po.make_inputs(1, 200, 2, 32, 32, seed=9, dtype=torch.bfloat16), gpu_device)
    cu = torch.from_numpy(ref["cu"]).to(gpu_device)
    a = (d["q"], d["k"], d["v"], d["b"], d["gt"], d["g"], d["Ip"])
    o_r, mu_r, I_r = fused_recurrent_palimpsa(*a, output_final_state=True, cu_seqlens=cu)
    o_c, mu_c, I_c = chunk_palimpsa(*a, output_final_state=True, cu_seqlens=cu, chunk_size=64)
    o_ref = torch.from_numpy(ref["o"])
    assert hp.max_abs(o_r, o_ref) <= hp.BF16_OUT_ABS_TOL and hp.max_abs(o_c, o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu_r, torch.from_numpy(ref["final_mu"])) <= hp.FP32_REL_TOL
    assert hp.max_rel(I_r, torch.from_numpy(ref["final_I"])) <= hp.FP32_REL_TOL
    assert hp.max_rel(mu_c, torch.from_numpy(ref["final_mu"])) <= 1e-2
    assert hp.max_rel(I_c, torch.from_numpy(ref["final_I"])) <= 1e-2


# ------------------------------------------------------------------ path without the precision state, layer glue
def test_oracles_reproduce_simple_gla_and_glue_fixtures():
    for name, case in (("simple_gla_grad.npz", mg.gla_case), ("layer_glue_grad.npz", mg.glue_case)):
        ref, now = _load(name), case()
        assert set(ref) == set(now)
        for k in ref:
            assert np.allclose(ref[k], now[k], rtol=1e-9, atol=1e-11), (name, k)


def test_simple_gla_fixture_against_dense_closed_form():
    """The stored vectors come from the recurrence oracle with b = 0; the same numbers follow from the dense form
    o = scale ((Q K^T) o L) V + scale F (Q S_0), which shares no code with it."""
    ref = _load("simple_gla_grad.npz")
    q, k, v, g, S0, _ = (x.double() for x in mg.gla_inputs())
    c = g.cumsum(1)
    T = q.shape[1]
    Lm = torch.exp(c[:, :, None] - c[:, None, :]) * torch.tril(torch.ones(T, T, dtype=torch.float64))[None, :, :, None]
    o = torch.einsum("bthn,bshn,btsh,bshd->bthd", q, k, Lm, v) + torch.einsum("bthn,bth,bhnd->bthd", q, torch.exp(c), S0)
    assert np.allclose(ref["o"], (0.25 * o).numpy(), rtol=1e-9, atol=1e-11)
    S = torch.einsum("bshn,bsh,bshd->bhnd", k, torch.exp(c[:, -1:] - c), v) + torch.exp(c[:, -1])[..., None, None] * S0
    assert np.allclose(ref["final_state"], S.numpy(), rtol=1e-9, atol=1e-11)


@pytest.mark.gpu
def test_gpu_simple_gla_hits_fixture(gpu_device):
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla, fused_recurrent_simple_gla

    ref = _load("simple_gla_grad.npz")
    q, k, v, g, S0, do = mg.gla_inputs()
    dev = gpu_device
    leaves = [x.to(dev).clone().requires_grad_(True) for x in (q, k, v, g, S0)]
    o, S = chunk_simple_gla(q=leaves[0], k=leaves[1], v=leaves[2], g=leaves[3], scale=0.25, initial_state=leaves[4],
                            output_final_state=True)
    (o.float() * do.to(dev)).sum().backward()
    assert hp.max_abs(o.float(), torch.from_numpy(ref["o"])) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(S, torch.from_numpy(ref["final_state"])) <= 1e-2
    for n, x in zip(("q", "k", "v", "g", "S0"), leaves):
        assert hp.max_rel(x.grad, torch.from_numpy(ref["d" + n])) <= hp.BF16_GRAD_NORM_TOL, n
    with torch.no_grad():
        o_r, S_r = fused_recurrent_simple_gla(q=q.to(dev), k=k.to(dev), v=v.to(dev), g=g.to(dev), scale=0.25,
                                              initial_state=S0.to(dev), output_final_state=True)
    assert hp.max_abs(o_r.float(), torch.from_numpy(ref["o"])) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(S_r, torch.from_numpy(ref["final_state"])) <= hp.FP32_REL_TOL


@pytest.mark.gpu
def test_gpu_layer_glue_hits_fixture(gpu_device):
    from palimpsa_amd.ops.layer_glue import palimpsa_inputs, palimpsa_output_norm

    ref = _load("layer_glue_grad.npz")
    a, extra, wts = mg.glue_inputs()
    dev = gpu_device
    names = list(a)
    leaves = {n: a[n].to(dev).clone().requires_grad_(True) for n in names}
    outs = palimpsa_inputs(**leaves)
    loss = sum((y.float() * w.to(dev)).sum() for y, w in zip(outs, wts))
    loss.backward()
    for n, y in zip(("q", "k", "v", "b", "gt"), outs):
        r = torch.from_numpy(ref["pro_" + n])
        assert hp.max_abs(y.float(), r) <= hp.BF16_OUT_ABS_TOL * max(1.0, r.abs().max().item()), n
    for n in names:
        assert hp.max_rel(leaves[n].grad, torch.from_numpy(ref["pro_d" + n])) <= hp.BF16_GRAD_NORM_TOL, n
    ev = [extra["o"], a["x"], extra["D"], extra["gate"], extra["weight"]]
    lv = [t.to(dev).clone().requires_grad_(True) for t in ev]
    y = palimpsa_output_norm(*lv, 1e-6)
    y.backward(extra["dy"].to(dev))
    r = torch.from_numpy(ref["epi_y"])
    assert hp.max_abs(y.float(), r) <= hp.BF16_OUT_ABS_TOL * max(1.0, r.abs().max().item())
    for n, t in zip(("o", "x", "D", "gate", "weight"), lv):
        assert hp.max_rel(t.grad, torch.from_numpy(ref["epi_d" + n])) <= hp.BF16_GRAD_NORM_TOL, n
