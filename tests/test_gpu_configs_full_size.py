"""The larger benchmark configurations at their full shapes on the GPU.

The CPU oracle checks a subset that it finishes in seconds (documents, heads and sequences are
independent, so a slice of the inputs is a complete problem of its own); the whole result is
checked through properties that do not depend on the size: the chunked kernels against the
fp32-state token-serial kernel (a second, independent implementation), split/resume through the
state, and the identity dg = sum_t gt_t dgt_t / g that ties the per-head reduction to the
per-token gate gradients.

  c2  packed documents, 32768 tokens, H=16, dk=dv=96, bf16, chunked forward + backward
  c3  decode, B=256, H=16, dk=dv=128, bf16 rows, fp32 states fed back step after step
  c4  prefill, T=65536, H=16, dk=dv=128, bf16, chunked forward with initial and final state
"""
import pytest
import torch

from oracle import palimpsa_oracle as po
from tests import helpers as hp

pytestmark = pytest.mark.gpu
STATE_REL_TOL = 1e-2


def _ops():
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa, fused_recurrent_palimpsa
    return chunk_palimpsa, fused_recurrent_palimpsa


def test_c2_packed_documents_forward_backward(gpu_device):
    ck, fr = _ops()
    cu = po.make_varlen_lengths(32768, seed=0)
    T, H, d = cu[-1], 16, 96
    assert T == 32768
    inp = hp.rounded(po.make_inputs(1, T, H, d, d, seed=0), torch.bfloat16)
    gen = torch.Generator().manual_seed(1)
    do = torch.randn(1, T, H, d, generator=gen)
    dev = gpu_device
    leaves = {n: inp[n].to(dev).clone().requires_grad_(True) for n in ("q", "k", "v", "b", "gt", "g", "Ip")}
    cu_d = torch.tensor(cu, device=dev, dtype=torch.int32)
    o = ck(*[leaves[n] for n in ("q", "k", "v", "b", "gt", "g", "Ip")], chunk_size=64, cu_seqlens=cu_d)
    (o.float() * do.to(dev)).sum().backward()
    grads = {n: x.grad for n, x in leaves.items()}
    for n, x in grads.items():
        assert torch.isfinite(x.float()).all(), n

    # whole forward against the token-serial fp32-state kernel
    with torch.no_grad():
        o_r = fr(*[leaves[n] for n in ("q", "k", "v", "b", "gt", "g", "Ip")], cu_seqlens=cu_d)
    assert hp.max_abs(o.float(), o_r.float()) <= hp.BF16_OUT_ABS_TOL

    # the per-head reduction is consistent with the per-token gate gradients over all 32768 tokens
    dg_from_dgt = (inp["gt"].double() * grads["gt"].double().cpu()).sum(dim=(0, 1)) / inp["g"].double()
    mass = (inp["gt"].double() * grads["gt"].double().cpu()).abs().sum(dim=(0, 1)) / inp["g"].double()
    assert ((grads["g"].double().cpu() - dg_from_dgt).abs() / mass).max().item() <= 1e-3

    # oracle (float64, autograd) on three documents and two heads
    hs = [3, 12]
    lens = [cu[j + 1] - cu[j] for j in range(len(cu) - 1)]
    order = sorted(range(len(lens)), key=lambda j: lens[j])
    small = [j for j in order if lens[j] <= 1024]   # float64 autograd through the oracle keeps every step
    docs = [small[0], small[len(small) // 2], small[-1]]
    for j in docs:
        sl = slice(cu[j], cu[j + 1])
        sub = {n: inp[n][:, sl][:, :, hs] for n in ("q", "k", "v", "b", "gt")}
        sub["g"], sub["Ip"] = inp["g"][hs], inp["Ip"][hs]
        ref = hp.oracle_grads(sub, do[:, sl][:, :, hs])
        assert hp.max_abs(o[:, sl][:, :, hs].float(), ref["o"]) <= hp.BF16_OUT_ABS_TOL
        for n in ("q", "k", "v", "b", "gt"):
            err = hp.max_rel(grads[n][:, sl][:, :, hs], ref[n])
            assert err <= hp.BF16_GRAD_NORM_TOL, (j, n, err)

    # the per-head reductions dg, dIp over ALL documents (the kernel sums 22 documents' shares per head): the oracle
    # runs every document of one head with autograd (float64, document by document so that only one document's
    # per-token states are alive at a time) and its gradients are added up.  dg is normalised by the l1 mass of its
    # terms (random dO: |dg| is far below the sum of the magnitudes, see tests/test_gpu_chunk_bwd.py), dIp likewise by
    # the mass of its per-document terms.
    h = 12
    dg_ref = dIp_ref = 0.0
    dg_mass = dIp_mass = 0.0
    for j in range(len(cu) - 1):
        sl = slice(cu[j], cu[j + 1])
        sub = {n: inp[n][:, sl][:, :, [h]] for n in ("q", "k", "v", "b", "gt")}
        sub["g"], sub["Ip"] = inp["g"][[h]], inp["Ip"][[h]]
        ref = hp.oracle_grads(sub, do[:, sl][:, :, [h]])
        dg_ref += ref["g"].item()
        dIp_ref += ref["Ip"].item()
        dg_mass += (sub["gt"].double() * ref["gt"].double()).abs().sum().item() / sub["g"].item()
        dIp_mass += abs(ref["Ip"].item())
    e_g = abs(grads["g"][h].item() - dg_ref) / dg_mass
    e_Ip = abs(grads["Ip"][h].item() - dIp_ref) / dIp_mass
    print(f"c2 head {h}: dg {grads['g'][h].item():.5e} ref {dg_ref:.5e} |d|/mass {e_g:.2e}; "
          f"dIp {grads['Ip'][h].item():.5e} ref {dIp_ref:.5e} |d|/mass {e_Ip:.2e}")
    assert e_g <= hp.BF16_GRAD_NORM_TOL and e_Ip <= hp.BF16_GRAD_NORM_TOL


def test_c3_decode_steps_with_state_fed_back(gpu_device):
    _, fr = _ops()
    B, H, d, steps = 256, 16, 128, 16
    dev = gpu_device
    inp = hp.rounded(po.make_inputs(B, steps, H, d, d, seed=0), torch.bfloat16)
    gen = torch.Generator().manual_seed(3)
    mu0 = torch.randn(B, H, d, d, generator=gen) * 0.1
    I0 = torch.nn.functional.softplus(torch.randn(B, H, d, d, generator=gen))
    dv_ = hp.to_device(inp, dev)
    mu, I = mu0.to(dev), I0.to(dev)
    outs = []
    for t in range(steps):
        r = {n: dv_[n][:, t:t + 1].contiguous() for n in ("q", "k", "v", "b", "gt")}
        o, mu, I = fr(r["q"], r["k"], r["v"], r["b"], r["gt"], dv_["g"], dv_["Ip"],
                      initial_mu_state=mu, initial_I_state=I, output_final_state=True)
        outs.append(o)
    o_steps = torch.cat(outs, dim=1)
    # 16 single-token calls == one 16-token call from the same state (full width)
    o_one, mu_one, I_one = fr(dv_["q"], dv_["k"], dv_["v"], dv_["b"], dv_["gt"], dv_["g"], dv_["Ip"],
                              initial_mu_state=mu0.to(dev), initial_I_state=I0.to(dev), output_final_state=True)
    # (the state crosses every call boundary as (mu, I) = (M / I, I): one fp32 rounding per step, and the
    #  bf16 outputs may differ in their last bit)
    assert hp.max_abs(o_steps.float(), o_one.float()) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu, mu_one) <= 1e-5 and hp.max_rel(I, I_one) <= 1e-5
    # oracle on a subset of sequences
    bs = [0, 101, 255]
    sub = {n: inp[n][bs] for n in ("q", "k", "v", "b", "gt")}
    sub["g"], sub["Ip"] = inp["g"], inp["Ip"]
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(sub, mu0=mu0[bs], I0=I0[bs])
    assert hp.max_abs(o_steps[bs].float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu[bs], mu_ref) <= hp.FP32_REL_TOL
    assert hp.max_rel(I[bs], I_ref) <= hp.FP32_REL_TOL


def test_c4_long_prefill_with_states(gpu_device):
    ck, fr = _ops()
    T, H, d = 65536, 16, 128
    dev = gpu_device
    inp = hp.rounded(po.make_inputs(1, T, H, d, d, seed=0), torch.bfloat16)
    gen = torch.Generator().manual_seed(3)
    mu0 = torch.randn(1, H, d, d, generator=gen) * 0.1
    I0 = inp["Ip"].view(1, H, 1, 1) + torch.nn.functional.softplus(torch.randn(1, H, d, d, generator=gen))
    dv_ = hp.to_device(inp, dev)
    args = [dv_[n] for n in ("q", "k", "v", "b", "gt", "g", "Ip")]
    with torch.no_grad():
        o, mu, I = ck(*args, chunk_size=64, initial_mu_state=mu0.to(dev), initial_I_state=I0.to(dev),
                      output_final_state=True)
        # second implementation, whole tensor
        o_r, mu_r, I_r = fr(*args, initial_mu_state=mu0.to(dev), initial_I_state=I0.to(dev), output_final_state=True)
        # split / resume: two halves through the state reproduce the single call
        half = T // 2
        a1 = [dv_[n][:, :half].contiguous() for n in ("q", "k", "v", "b", "gt")] + [dv_["g"], dv_["Ip"]]
        a2 = [dv_[n][:, half:].contiguous() for n in ("q", "k", "v", "b", "gt")] + [dv_["g"], dv_["Ip"]]
        o1, m1, i1 = ck(*a1, chunk_size=64, initial_mu_state=mu0.to(dev), initial_I_state=I0.to(dev), output_final_state=True)
        o2, m2, i2 = ck(*a2, chunk_size=64, initial_mu_state=m1, initial_I_state=i1, output_final_state=True)
    assert torch.isfinite(o.float()).all()
    assert hp.max_abs(o.float(), o_r.float()) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu, mu_r) <= STATE_REL_TOL and hp.max_rel(I, I_r) <= STATE_REL_TOL
    assert hp.max_abs(torch.cat([o1, o2], dim=1).float(), o.float()) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(m2, mu) <= 1e-5 and hp.max_rel(i2, I) <= 1e-5
    # oracle on one head over all 65536 tokens
    hs = [9]
    sub = {n: inp[n][:, :, hs] for n in ("q", "k", "v", "b", "gt")}
    sub["g"], sub["Ip"] = inp["g"][hs], inp["Ip"][hs]
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(sub, mu0=mu0[:, hs], I0=I0[:, hs])
    assert hp.max_abs(o[:, :, hs].float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu[:, hs], mu_ref) <= STATE_REL_TOL
    assert hp.max_rel(I[:, hs], I_ref) <= STATE_REL_TOL
