"""Tensors of more than 2^31 elements (more than 4 GiB): every element offset in the kernels is 64-bit.

A GPU with 288 GB holds row tensors and decode states far beyond the range of a 32-bit index.  The
shapes here put the last sequences of a batch beyond element 2^31 of q, k, v, b, o (and of the
gradients), and the last sequences of a decode batch beyond byte 2^32 of the state tensors.
Sequences are independent, so the result for the last sequences has to be what a call on those
sequences alone returns; the whole output is also compared with the second implementation
(chunked against token-serial), which walks the same tensors with different index arithmetic.
"""
import pytest
import torch
import torch.nn.functional as F

from tests import helpers as hp

pytestmark = pytest.mark.gpu

ROW_NAMES = ("q", "k", "v", "b", "gt")


def _rows(B, T, H, d, dev, gen, fn, dtype=torch.bfloat16, slab=16):
    """[B,T,H,d] rows generated slab by slab (the fp32 temporaries stay small)."""
    out = torch.empty(B, T, H, d, dtype=dtype, device=dev)
    for b0 in range(0, B, slab):
        n = min(slab, B - b0)
        out[b0:b0 + n] = fn(torch.randn(n, T, H, d, generator=gen, device=dev)).to(dtype)
    return out


def _inputs(B, T, H, dk, dv, dev, seed):
    gen = torch.Generator(device=dev).manual_seed(seed)
    inp = {
        "q": _rows(B, T, H, dk, dev, gen, lambda x: F.normalize(x, dim=-1)),
        "k": _rows(B, T, H, dk, dev, gen, lambda x: F.normalize(x, dim=-1)),
        "v": _rows(B, T, H, dv, dev, gen, lambda x: x),
        "b": _rows(B, T, H, dv, dev, gen, torch.sigmoid),
        "gt": torch.sigmoid(torch.randn(B, T, H, generator=gen, device=dev)),
        "g": torch.ones(H, device=dev),
        "Ip": torch.ones(H, device=dev),
    }
    return inp, gen


def _max_abs_slabs(x, y, slab=16):
    """max |x - y| over tensors too large for an fp32 temporary of their full size."""
    worst = 0.0
    for b0 in range(0, x.shape[0], slab):
        worst = max(worst, (x[b0:b0 + slab].float() - y[b0:b0 + slab].float()).abs().max().item())
    return worst


def test_chunked_forward_backward_beyond_2_31_elements(gpu_device):
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa, fused_recurrent_palimpsa
    dev = gpu_device
    B, T, H, d = 288, 8192, 16, 64
    assert B * T * H * d > 2 ** 31 + 2 ** 27           # the last sequences lie beyond element 2^31
    inp, gen = _inputs(B, T, H, d, d, dev, seed=11)
    do = _rows(B, T, H, d, dev, gen, lambda x: x)
    leaves = {n: inp[n].requires_grad_(True) for n in ROW_NAMES + ("g", "Ip")}
    args = [leaves[n] for n in ROW_NAMES + ("g", "Ip")]
    o = chunk_palimpsa(*args, chunk_size=64)
    o.backward(do)
    grads = {n: leaves[n].grad for n in ROW_NAMES}
    assert torch.isfinite(leaves["g"].grad).all() and torch.isfinite(leaves["Ip"].grad).all()

    # the whole output against the token-serial kernel
    with torch.no_grad():
        o_rec = fused_recurrent_palimpsa(*args)
    assert _max_abs_slabs(o, o_rec) <= hp.BF16_OUT_ABS_TOL
    del o_rec

    # first, middle and last sequences on their own (the last two start beyond element 2^31 / 2 and 2^31)
    sel = [0, B // 2 + 1, B - 2, B - 1]
    sub = {n: leaves[n].detach()[sel].clone().requires_grad_(True) for n in ROW_NAMES}
    sub["g"] = leaves["g"].detach().clone().requires_grad_(True)
    sub["Ip"] = leaves["Ip"].detach().clone().requires_grad_(True)
    o_s = chunk_palimpsa(*[sub[n] for n in ROW_NAMES + ("g", "Ip")], chunk_size=64)
    o_s.backward(do[sel].clone())
    assert hp.max_abs(o.detach()[sel].float(), o_s.detach().float()) <= 1e-6
    for n in ROW_NAMES:
        ref = sub[n].grad.float()
        err = (grads[n][sel].float() - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)
        assert err <= 1e-6, (n, err)


def test_packed_documents_beyond_2_31_elements(gpu_device):
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa, fused_recurrent_palimpsa
    dev = gpu_device
    T, H, d = 288 * 8192, 16, 64
    # documents of 5000 to 60000 tokens, the last ones beyond element 2^31 of the packed rows
    lens, tot, j = [], 0, 0
    while tot < T:
        ln = min(5000 + (j * 7919) % 55000, T - tot)
        lens.append(ln)
        tot += ln
        j += 1
    cu = [0]
    for ln in lens:
        cu.append(cu[-1] + ln)
    inp, gen = _inputs(1, T, H, d, d, dev, seed=12)
    cu_d = torch.tensor(cu, device=dev, dtype=torch.int32)
    args = [inp[n] for n in ROW_NAMES + ("g", "Ip")]
    with torch.no_grad():
        o = chunk_palimpsa(*args, chunk_size=64, cu_seqlens=cu_d)
        o_rec = fused_recurrent_palimpsa(*args, cu_seqlens=cu_d)
    worst = 0.0
    for t0 in range(0, T, 1 << 17):
        worst = max(worst, (o[:, t0:t0 + (1 << 17)].float() - o_rec[:, t0:t0 + (1 << 17)].float()).abs().max().item())
    assert worst <= hp.BF16_OUT_ABS_TOL
    # the last document on its own
    sl = slice(cu[-2], cu[-1])
    with torch.no_grad():
        o_last = chunk_palimpsa(*[inp[n][:, sl].contiguous() for n in ROW_NAMES], inp["g"], inp["Ip"], chunk_size=64)
    assert hp.max_abs(o[:, sl].float(), o_last.float()) <= 1e-6


def test_decode_states_beyond_4_gib(gpu_device):
    from palimpsa_amd.ops.palimpsa import DecodeStep, fused_recurrent_palimpsa
    dev = gpu_device
    B, H, d = 4352, 16, 128
    assert B * H * d * d * 4 > 2 ** 32 + 2 ** 27        # fp32 state tensors of 4.25 GiB each
    gen = torch.Generator(device=dev).manual_seed(13)
    mu = torch.empty(B, H, d, d, device=dev)
    I = torch.empty(B, H, d, d, device=dev)
    for b0 in range(0, B, 256):
        mu[b0:b0 + 256] = torch.randn(256, H, d, d, generator=gen, device=dev) * 0.1
        I[b0:b0 + 256] = 1.0 + F.softplus(torch.randn(256, H, d, d, generator=gen, device=dev))
    inp, _ = _inputs(B, 1, H, d, d, dev, seed=14)
    sel = [0, B // 2 + 1, B - 1]
    mu_s, I_s = mu[sel].clone(), I[sel].clone()
    step = DecodeStep(B, H, d, d, dev).bind(inp["q"], inp["k"], inp["v"], inp["b"], inp["gt"], inp["g"], inp["Ip"], mu, I)
    o = step.step().clone()
    o_s, mu_r, I_r = fused_recurrent_palimpsa(*[inp[n][sel].contiguous() for n in ROW_NAMES], inp["g"], inp["Ip"],
                                              initial_mu_state=mu_s, initial_I_state=I_s, output_final_state=True)
    assert torch.equal(o[sel], o_s)
    assert torch.equal(mu[sel], mu_r) and torch.equal(I[sel], I_r)
    # a second step from the updated state, through the entry point with separate state tensors
    o2, mu2, I2 = fused_recurrent_palimpsa(*[inp[n] for n in ROW_NAMES], inp["g"], inp["Ip"],
                                           initial_mu_state=mu, initial_I_state=I, output_final_state=True)
    o2_s, mu2_r, I2_r = fused_recurrent_palimpsa(*[inp[n][sel].contiguous() for n in ROW_NAMES], inp["g"], inp["Ip"],
                                                 initial_mu_state=mu_r, initial_I_state=I_r, output_final_state=True)
    assert torch.equal(o2[sel], o2_s)
    assert torch.equal(mu2[sel], mu2_r) and torch.equal(I2[sel], I2_r)


def test_scalar_gated_forward_backward_beyond_2_31_elements(gpu_device):
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla, fused_recurrent_simple_gla
    dev = gpu_device
    B, T, H, d = 288, 8192, 16, 64
    gen = torch.Generator(device=dev).manual_seed(15)
    q = _rows(B, T, H, d, dev, gen, lambda x: F.normalize(x, dim=-1)).requires_grad_(True)
    k = _rows(B, T, H, d, dev, gen, lambda x: F.normalize(x, dim=-1)).requires_grad_(True)
    v = _rows(B, T, H, d, dev, gen, lambda x: x).requires_grad_(True)
    g = (-torch.sigmoid(torch.randn(B, T, H, generator=gen, device=dev))).requires_grad_(True)
    do = _rows(B, T, H, d, dev, gen, lambda x: x)
    o = chunk_simple_gla(q, k, v, g)
    o = o[0] if isinstance(o, tuple) else o
    o.backward(do)
    with torch.no_grad():
        o_rec = fused_recurrent_simple_gla(q, k, v, g)
        o_rec = o_rec[0] if isinstance(o_rec, tuple) else o_rec
    assert _max_abs_slabs(o, o_rec) <= hp.BF16_OUT_ABS_TOL
    del o_rec
    sel = [0, B // 2 + 1, B - 1]
    sub = [x.detach()[sel].clone().requires_grad_(True) for x in (q, k, v, g)]
    o_s = chunk_simple_gla(*sub)
    o_s = o_s[0] if isinstance(o_s, tuple) else o_s
    o_s.backward(do[sel].clone())
    assert hp.max_abs(o.detach()[sel].float(), o_s.detach().float()) <= 1e-6
    for name, full, part in zip("qkvg", (q, k, v, g), sub):
        ref = part.grad.float()
        err = (full.grad[sel].float() - ref).abs().max().item() / max(ref.abs().max().item(), 1e-30)
        assert err <= 1e-6, (name, err)


def test_layer_glue_beyond_2_31_elements(gpu_device):
    from palimpsa_amd.ops.layer_glue import palimpsa_inputs, palimpsa_output_norm
    dev = gpu_device
    B, T, H, d = 288, 8192, 16, 64
    gen = torch.Generator(device=dev).manual_seed(16)
    big = {n: _rows(B, T, H, d, dev, gen, lambda x: x) for n in ("q_raw", "k_raw", "x", "b_raw", "gate")}
    big["dt_raw"] = torch.randn(B, T, H, generator=gen, device=dev).to(torch.bfloat16)
    big["bs_raw"] = torch.randn(B, T, H, generator=gen, device=dev).to(torch.bfloat16)
    par = {"dt_bias": torch.randn(H, generator=gen, device=dev), "b_scale": torch.randn(H, generator=gen, device=dev),
           "D": torch.randn(H, generator=gen, device=dev), "weight": 1.0 + 0.1 * torch.randn(d, generator=gen, device=dev)}
    seeds = [_rows(B, T, H, d, dev, gen, lambda x: x) for _ in range(2)]     # gradients of v and of the normed output
    sel = [0, B // 2 + 1, B - 1]

    def run(t, p, s):
        t = {n: x.detach().clone().requires_grad_(True) for n, x in t.items()}
        p = {n: x.detach().clone().requires_grad_(True) for n, x in p.items()}
        q, k, v, b, gt = palimpsa_inputs(t["q_raw"], t["k_raw"], t["x"], t["dt_raw"], p["dt_bias"], t["bs_raw"],
                                         t["b_raw"], p["b_scale"])
        y = palimpsa_output_norm(v, t["x"], p["D"], t["gate"], p["weight"])
        torch.autograd.backward([v, y, q, k, b, gt], [s[0], s[1], s[0], s[1], s[1], torch.ones_like(gt)])
        return {"q": q, "k": k, "v": v, "b": b, "gt": gt, "y": y}, {n: x.grad for n, x in t.items()}, \
               {n: x.grad for n, x in p.items()}

    out, gr, gp = run(big, par, seeds)
    for n, x in gp.items():
        assert torch.isfinite(x).all(), n
    out_s, gr_s, _ = run({n: x[sel] for n, x in big.items()}, par, [s[sel] for s in seeds])
    for n in out:
        assert torch.equal(out[n].detach()[sel], out_s[n].detach()), n
    for n in gr:
        assert torch.equal(gr[n][sel], gr_s[n]), n
