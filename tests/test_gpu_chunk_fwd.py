"""GPU parity of the chunked forward (bf16 MFMA kernels) against the CPU oracle.

Calls go through palimpsa_amd.ops.palimpsa.chunk_palimpsa -> ctypes -> C ABI.
The chunked kernels contract in bf16 on the matrix cores whatever the input
dtype, so their bar is the bf16 one: max|o - ref| <= 2e-2 with the oracle fed
the same rounded rows.  Final states accumulate bf16-rounded products in fp32:
max|x-ref|/max|ref| <= 1e-2.
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


def _call(fn, d, **kw):
    return fn(d["q"], d["k"], d["v"], d["b"], d["gt"], d["g"], d["Ip"], **kw)


@pytest.mark.parametrize("T", [1, 63, 64, 65, 200])
def test_bf16_forward_lengths(gpu_device, T):
    ck, _ = _ops()
    inp = hp.rounded(po.make_inputs(2, T, 3, 64, 64, seed=T), torch.bfloat16)
    inp["g"] = torch.tensor([1.0, 4.0, 0.25])
    o_ref, ov_ref, mu_ref, I_ref = hp.oracle_forward(inp, want_var=True)
    d = hp.to_device(inp, gpu_device)
    (o, ov), mu, I = _call(ck, d, output_final_state=True, output_uncertainty=True, chunk_size=64)
    assert o.dtype == torch.bfloat16 and ov.dtype == torch.bfloat16
    assert hp.max_abs(o, o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_abs(ov, ov_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu, mu_ref) <= STATE_REL_TOL
    assert hp.max_rel(I, I_ref) <= STATE_REL_TOL


@pytest.mark.parametrize("dk,dv", [(16, 16), (32, 32), (48, 96), (96, 96), (128, 128), (64, 192), (256, 32), (31, 65)])
def test_bf16_forward_head_dims_with_initial_state(gpu_device, dk, dv):
    ck, _ = _ops()
    B, T, H = 2, 130, 2
    inp = hp.rounded(po.make_inputs(B, T, H, dk, dv, seed=dk * 3 + dv), torch.bfloat16)
    inp["Ip"] = torch.tensor([0.5, 2.0])
    gen = torch.Generator().manual_seed(2)
    mu0 = torch.randn(B, H, dv, dk, generator=gen) * 0.1
    I0 = inp["Ip"].view(1, H, 1, 1) + torch.nn.functional.softplus(torch.randn(B, H, dv, dk, generator=gen))
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(inp, scale=0.5, mu0=mu0, I0=I0)
    d = hp.to_device(inp, gpu_device)
    o, mu, I = _call(ck, d, scale=0.5, initial_mu_state=mu0.to(gpu_device), initial_I_state=I0.to(gpu_device),
                     output_final_state=True)
    assert o.shape == (B, T, H, dv) and mu.shape == (B, H, dv, dk)
    assert hp.max_abs(o, o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu, mu_ref) <= STATE_REL_TOL
    assert hp.max_rel(I, I_ref) <= STATE_REL_TOL


@pytest.mark.parametrize("dk,dv", [(32, 48), (64, 64), (96, 192), (128, 128), (256, 256), (31, 65)])
def test_fp32_inputs_meet_the_fp32_bar(gpu_device, dk, dv):
    """fp32 rows take the split-operand variants of the chunked kernels: outputs, uncertainty and final states within
    1e-4 (relative, max-norm) of the float64 oracle at every head dim, 256 x 256 included (value rows then go
    through the tile-state kernel in pieces)."""
    ck, _ = _ops()
    B, T, H = 2, 200, 2
    inp = po.make_inputs(B, T, H, dk, dv, seed=4)
    inp["g"] = torch.tensor([0.7, 6.0])
    inp["Ip"] = torch.tensor([0.4, 1.7])
    gen = torch.Generator().manual_seed(8)
    mu0 = torch.randn(B, H, dv, dk, generator=gen) * 0.1
    I0 = inp["Ip"].view(1, H, 1, 1) + torch.nn.functional.softplus(torch.randn(B, H, dv, dk, generator=gen))
    o_ref, ov_ref, mu_ref, I_ref = hp.oracle_forward(inp, mu0=mu0, I0=I0, want_var=True, dtype=torch.float64)
    d = hp.to_device(inp, gpu_device)
    (o, ov), mu, I = _call(ck, d, initial_mu_state=mu0.to(gpu_device), initial_I_state=I0.to(gpu_device),
                           output_final_state=True, output_uncertainty=True)
    assert o.dtype == torch.float32
    for x, r in ((o, o_ref), (ov, ov_ref), (mu, mu_ref), (I, I_ref)):
        assert hp.max_rel(x, r) <= hp.FP32_REL_TOL


def test_fp32_fast_mode_is_an_opt_in_at_bf16_accuracy(gpu_device):
    """PAL_FLAG_FP32_FAST (here through the Python knob): fp32 rows rounded to single bf16/f16 operands, the accuracy
    of the bf16 path, about twice as fast; never the default."""
    from palimpsa_amd import _lib
    ck, _ = _ops()
    inp = po.make_inputs(2, 100, 2, 32, 48, seed=4)
    o_ref, _, _, _ = hp.oracle_forward(inp, dtype=torch.float64)
    d = hp.to_device(inp, gpu_device)
    try:
        _lib.set_fp32_fast(True)
        o_fast = _call(ck, d)
    finally:
        _lib.set_fp32_fast(False)
    o = _call(ck, d)
    assert o_fast.dtype == torch.float32
    e_fast, e = hp.max_rel(o_fast, o_ref), hp.max_rel(o, o_ref)
    assert e <= hp.FP32_REL_TOL < e_fast <= hp.BF16_OUT_ABS_TOL


def test_varlen_equals_per_document_oracle(gpu_device):
    ck, _ = _ops()
    H, dk, dv = 2, 64, 64
    cu = [0, 1, 65, 129, 130, 330, 400]
    T, N = cu[-1], len(cu) - 1
    inp = hp.rounded(po.make_inputs(1, T, H, dk, dv, seed=7), torch.bfloat16)
    gen = torch.Generator().manual_seed(3)
    mu0 = torch.randn(N, H, dv, dk, generator=gen) * 0.1
    I0 = 1.0 + torch.rand(N, H, dv, dk, generator=gen)
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(inp, mu0=mu0, I0=I0, cu=cu)
    d = hp.to_device(inp, gpu_device)
    o, mu, I = _call(ck, d, initial_mu_state=mu0.to(gpu_device), initial_I_state=I0.to(gpu_device),
                     output_final_state=True, cu_seqlens=torch.tensor(cu, device=gpu_device))
    assert hp.max_abs(o, o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu, mu_ref) <= STATE_REL_TOL
    assert hp.max_rel(I, I_ref) <= STATE_REL_TOL
    # no initial state: every document restarts from (0, Ip)
    o_ref2, _, _, _ = hp.oracle_forward(inp, cu=cu)
    o2 = _call(ck, d, cu_seqlens=torch.tensor(cu, device=gpu_device))
    assert hp.max_abs(o2, o_ref2) <= hp.BF16_OUT_ABS_TOL


@pytest.mark.parametrize("gate_dtype", [None, torch.bfloat16], ids=["fp32_gates", "bf16_gates"])
def test_c1_shape_subset_against_oracle_and_full_against_recurrent(gpu_device, gate_dtype):
    """Config 1 (B=8,T=2048,H=12,d=64,bf16): the oracle checks a (batch, head) subset at full T
    (entries are independent); the whole tensor is checked against the fp32-state recurrent kernel.
    With bf16 gates (the gate tensor handed over in bf16, as config 1 says and bench.py times) the oracle is fed
    the same rounded gates."""
    ck, fr = _ops()
    inp = hp.rounded(po.make_inputs(8, 2048, 12, 64, 64, seed=0), torch.bfloat16)
    d = hp.to_device(inp, gpu_device)
    if gate_dtype is not None:
        inp["gt"] = inp["gt"].to(gate_dtype).float()
        d["gt"] = d["gt"].to(gate_dtype)
    o, mu, I = _call(ck, d, output_final_state=True, chunk_size=64)
    o_r, mu_r, I_r = _call(fr, d, output_final_state=True)
    assert hp.max_abs(o.float(), o_r.float()) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu, mu_r) <= STATE_REL_TOL
    assert hp.max_rel(I, I_r) <= STATE_REL_TOL
    bs, hs = [0, 5], [1, 7, 11]
    sub = {n: inp[n][bs][:, :, hs] for n in ("q", "k", "v", "b", "gt")}
    sub["g"], sub["Ip"] = inp["g"][hs], inp["Ip"][hs]
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(sub)
    assert hp.max_abs(o[bs][:, :, hs], o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu[bs][:, hs], mu_ref) <= STATE_REL_TOL
    assert hp.max_rel(I[bs][:, hs], I_ref) <= STATE_REL_TOL


def test_error_paths_match_reference(gpu_device):
    ck, _ = _ops()
    inp = hp.to_device(po.make_inputs(2, 8, 2, 16, 16, seed=0), gpu_device)
    with pytest.raises(ValueError):
        _call(ck, inp, cu_seqlens=torch.tensor([0, 8], device=gpu_device))


@pytest.mark.parametrize("v_scale,k_scale", [(3.0e5, 1.0), (40.0, 30.0), (1.0e-4, 1.0), (1.0e-6, 1.0), (1.0e-8, 1.0),
                                             (1.0, 300.0), (1.0e20, 1.0e-3), (1.0e-20, 1.0e3)])
def test_block_exponent_of_the_f16_operands(gpu_device, v_scale, k_scale):
    """Rows far from O(1), in both directions: the output kernel's f16 operands are normalised per tile by block
    exponents of k, v and b, so the relative error is that of O(1) rows and nothing overflows or flushes
    (|k| = 300 squares to 9e4, beyond the f16 range without the exponent of k)."""
    ck, _ = _ops()
    B, T, H, d = 1, 200, 2, 64
    inp = po.make_inputs(B, T, H, d, d, seed=77)
    inp["v"] = inp["v"] * v_scale
    inp["b"] = inp["b"] * v_scale
    inp["k"] = inp["k"] * k_scale
    inp = hp.rounded(inp, torch.bfloat16)
    o, mu, I = _call(ck, hp.to_device(inp, gpu_device), output_final_state=True, chunk_size=64)
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(inp)
    assert torch.isfinite(o.float()).all()
    assert hp.max_rel(o, o_ref) <= 1e-2
    assert hp.max_rel(mu, mu_ref) <= STATE_REL_TOL and hp.max_rel(I, I_ref) <= STATE_REL_TOL


@pytest.mark.parametrize("d", [64, 96])
@pytest.mark.parametrize("case", ["rows_shrink", "large_initial_state", "precision_below_prior", "rows_grow"])
def test_tile_start_state_in_the_first_token_operands(gpu_device, d, case):
    """The output kernels add the tile-start state to the f16 operands of a tile's first token and make room for it in
    the block exponents.  Cases where the state and the rows of a tile are far apart, for both kernel layouts
    (d = 64: by key columns, d = 96: by value rows): rows that shrink by 1e5 half way (the state then dwarfs them),
    an initial state 1e4 above the rows, an initial precision far below the prior (I_t = (1 - F_t) Ip + F_t I_0 + ...
    has no cancelling term), rows that grow by 1e4 (the state is then small against them)."""
    ck, _ = _ops()
    B, T, H = 1, 320, 2
    inp = po.make_inputs(B, T, H, d, d, seed=123)
    inp["g"] = torch.tensor([0.01, 0.2])     # slow decay: the state outlives the tiles
    gen = torch.Generator().manual_seed(124)
    kw = {}
    if case == "rows_shrink":
        inp["v"][:, T // 2:] *= 1.0e-5
        inp["b"][:, T // 2:] *= 1.0e-5
    elif case == "rows_grow":
        inp["v"][:, T // 2:] *= 1.0e4
        inp["b"][:, T // 2:] *= 1.0e4
    elif case == "large_initial_state":
        kw = dict(mu0=torch.randn(B, H, d, d, generator=gen) * 30.0, I0=1.0 + 300.0 * torch.rand(B, H, d, d, generator=gen))
    else:
        kw = dict(mu0=torch.randn(B, H, d, d, generator=gen), I0=0.01 + 0.04 * torch.rand(B, H, d, d, generator=gen))
    inp = hp.rounded(inp, torch.bfloat16)
    dev_kw = {}
    if kw:
        dev_kw = dict(initial_mu_state=kw["mu0"].to(gpu_device), initial_I_state=kw["I0"].to(gpu_device))
    (o, ov), mu, I = _call(ck, hp.to_device(inp, gpu_device), output_final_state=True, output_uncertainty=True,
                           chunk_size=64, **dev_kw)
    o_ref, ov_ref, mu_ref, I_ref = hp.oracle_forward(inp, want_var=True, **kw)
    assert torch.isfinite(o.float()).all() and torch.isfinite(ov.float()).all()
    # per half of the sequence: the halves differ by orders of magnitude in two of the cases
    for sl in (slice(0, T // 2), slice(T // 2, T)):
        assert hp.max_rel(o[:, sl], o_ref[:, sl]) <= 1e-2
        assert hp.max_rel(ov[:, sl], ov_ref[:, sl]) <= 1e-2
    assert hp.max_rel(mu, mu_ref) <= STATE_REL_TOL and hp.max_rel(I, I_ref) <= STATE_REL_TOL


def test_windowed_no_grad_forward_equals_single_call(gpu_device, monkeypatch):
    """A single long sequence without autograd is run in windows of tiles through the state
    (no tile-start states for the whole sequence); same kernels, same tiles, so the results agree
    with the single call to within the fp32 rounding of the state hand-over."""
    from palimpsa_amd.ops.palimpsa import chunk as chunk_mod
    ck, _ = _ops()
    B, T, H, d = 1, 2500, 2, 32
    inp = hp.rounded(po.make_inputs(B, T, H, d, d, seed=5), torch.bfloat16)
    dvc = hp.to_device(inp, gpu_device)
    gen = torch.Generator().manual_seed(6)
    mu0 = (torch.randn(B, H, d, d, generator=gen) * 0.1).to(gpu_device)
    I0 = (1.0 + torch.rand(B, H, d, d, generator=gen)).to(gpu_device)
    kw = dict(initial_mu_state=mu0, initial_I_state=I0, output_final_state=True, output_uncertainty=True, chunk_size=64)
    monkeypatch.setattr(chunk_mod, "_WINDOW_STATE_BYTES", 16 * 2 * 4 * H * d * d)   # 16 tiles per window
    assert chunk_mod._window_tiles(H, d, d) == 16
    with torch.no_grad():
        (o_w, ov_w), mu_w, I_w = _call(ck, dvc, **kw)
    dvc["v"] = dvc["v"].clone().requires_grad_(True)     # autograd path: one call, all tile-start states kept
    (o_s, ov_s), mu_s, I_s = _call(ck, dvc, **kw)
    assert hp.max_abs(o_w.float(), o_s.float()) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_abs(ov_w.float(), ov_s.float()) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu_w, mu_s) <= 1e-5 and hp.max_rel(I_w, I_s) <= 1e-5
    o_ref, _, mu_ref, I_ref = hp.oracle_forward(inp, mu0=mu0.cpu(), I0=I0.cpu())
    assert hp.max_abs(o_w.float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu_w, mu_ref) <= STATE_REL_TOL


@pytest.mark.parametrize("dk,dv", [(256, 256), (128, 256), (208, 240)])
def test_largest_head_dims_forward(gpu_device, dk, dv):
    """The largest head dims the forward takes (bf16 rows; the staging tiles of the tile-state kernel are bf16)."""
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa
    B, T, H = 1, 130, 2
    inp = hp.rounded(po.make_inputs(B, T, H, dk, dv, seed=5), torch.bfloat16)
    dev = gpu_device
    d = hp.to_device(inp, dev)
    with torch.no_grad():
        (o, ov), mu, I = chunk_palimpsa(d["q"], d["k"], d["v"], d["b"], d["gt"], d["g"], d["Ip"], chunk_size=64,
                                        output_final_state=True, output_uncertainty=True)
    o_ref, ov_ref, mu_ref, I_ref = hp.oracle_forward(inp, want_var=True)
    assert hp.max_abs(o.float(), o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_abs(ov.float(), ov_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu, mu_ref) <= STATE_REL_TOL and hp.max_rel(I, I_ref) <= STATE_REL_TOL


@pytest.mark.parametrize("backend", ["eager", "aot_eager"])
@pytest.mark.parametrize("case", ["chunk_dense", "chunk_packed_state_var", "recurrent"])
def test_entry_points_compile_without_a_graph_break(gpu_device, backend, case):
    """torch.compile(fullgraph=True) over a function that calls the operators: the entry points hand the tracer
    opaque library ops with shape-only implementations and registered gradients (the reference's wrapper was
    written to be traceable, chunk...py:627-651), so there is no graph break; same values and gradients as eager
    (the same kernels run).  'eager' exercises the tracer, 'aot_eager' also the fake tensors and the traced
    backward; no code generation is involved in either."""
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa, fused_recurrent_palimpsa
    dev = gpu_device
    names = ("q", "k", "v", "b", "gt", "g", "Ip")
    extra = []
    if case == "chunk_dense":
        inp = hp.rounded(po.make_inputs(2, 100, 2, 32, 32, seed=8), torch.bfloat16)

        def f(q, k, v, b, gt, g, Ip):
            return (chunk_palimpsa(q * 1.0, k, v, b, gt, g, Ip, chunk_size=64).float() ** 2).sum()
    elif case == "chunk_packed_state_var":
        cu = torch.tensor([0, 70, 71, 200], device=dev)
        inp = hp.rounded(po.make_inputs(1, 200, 2, 31, 65, seed=9), torch.bfloat16)     # padded head dims as well
        gen = torch.Generator().manual_seed(1)
        mu0 = (torch.randn(3, 2, 65, 31, generator=gen) * 0.1).to(dev).requires_grad_(True)
        I0 = (1.0 + torch.rand(3, 2, 65, 31, generator=gen)).to(dev).requires_grad_(True)
        extra = [mu0, I0]

        def f(q, k, v, b, gt, g, Ip):
            (o, ov), fmu, fI = chunk_palimpsa(q, k, v * 1.0, b, gt, g, Ip, initial_mu_state=mu0, initial_I_state=I0,
                                              output_final_state=True, output_uncertainty=True, cu_seqlens=cu)
            return (o.float() ** 2).sum() + ov.float().sum() + fmu.detach().sum() * 0.0
    else:
        inp = po.make_inputs(2, 40, 2, 32, 48, seed=10)

        def f(q, k, v, b, gt, g, Ip):
            o, fmu, fI = fused_recurrent_palimpsa(q, k * 1.0, v, b, gt, g, Ip, output_final_state=True)
            return (o ** 2).sum() + fI.detach().sum() * 0.0

    def run(fn):
        leaves = [inp[n].to(dev).clone().requires_grad_(True) for n in names]
        for x in extra:
            x.grad = None
        out = fn(*leaves)
        out.backward()
        return [out.detach()] + [x.grad for x in leaves] + [x.grad.clone() for x in extra]

    eager = run(f)
    torch._dynamo.reset()
    compiled = run(torch.compile(f, backend=backend, fullgraph=True))
    for a, b_ in zip(eager, compiled):
        assert hp.max_rel(b_, a) <= 1e-6


def test_library_ops_pass_opcheck(gpu_device):
    """torch.library.opcheck on the four ops: schema, fake implementation against the real one, autograd registration."""
    from palimpsa_amd.ops.palimpsa import _custom_ops as ops
    dev = gpu_device
    inp = hp.to_device(hp.rounded(po.make_inputs(1, 70, 2, 16, 32, seed=3), torch.bfloat16), dev)
    q, k, v, b, gt, g, Ip = [inp[n] for n in ("q", "k", "v", "b", "gt", "g", "Ip")]
    tests = ("test_schema", "test_faketensor", "test_autograd_registration")
    torch.library.opcheck(ops.chunk_fwd, (q, k, v, b, gt, g, Ip, None, None, 0.25, True, None, 0), test_utils=tests)
    out = ops.chunk_fwd(q, k, v, b, gt, g, Ip, None, None, 0.25, False, None, 0)
    torch.library.opcheck(ops.chunk_bwd, (q, k, v, b, gt, g, Ip, None, None, 0.25, None, out[4], out[5],
                                          torch.ones_like(v), None, 0), test_utils=tests)
    torch.library.opcheck(ops.recurrent_fwd, (q, k, v, b, gt, g, Ip, None, None, 0.25, True, True, None), test_utils=tests)
    torch.library.opcheck(ops.recurrent_bwd, (q, k, v, b, gt, g, Ip, None, None, 0.25, None, torch.ones_like(v), None),
                          test_utils=tests)


@pytest.mark.parametrize("dk,dv", [(96, 64), (80, 48), (32, 32)])
def test_output_kernel_wave_layouts_with_uncertainty(gpu_device, dk, dv):
    """Head dims whose forward output kernel runs two waves per column block (dk = 80, 96) or two (tile, head) pairs
    per workgroup (dk = 32; 3 tiles x 3 heads = an odd number of pairs, so the last workgroup has a spare group)."""
    ck, _ = _ops()
    B, T, H = 1, 150, 3
    inp = hp.rounded(po.make_inputs(B, T, H, dk, dv, seed=dk + dv), torch.bfloat16)
    o_ref, ov_ref, mu_ref, I_ref = hp.oracle_forward(inp, want_var=True)
    d = hp.to_device(inp, gpu_device)
    (o, ov), mu, I = _call(ck, d, output_final_state=True, output_uncertainty=True)
    assert hp.max_abs(o, o_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_abs(ov, ov_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu, mu_ref) <= STATE_REL_TOL and hp.max_rel(I, I_ref) <= STATE_REL_TOL


@pytest.mark.parametrize("dk,dv,var", [(112, 112, False), (64, 96, True), (96, 192, False), (48, 80, True),
                                       (16, 64, False), (128, 128, True)])
def test_output_kernel_row_layout_slices_packed(gpu_device, dk, dv, var):
    """Head dims whose forward output kernel is laid out by value rows, with slices of unequal size (112 = 64 + 48,
    80 = 48 + 32 with uncertainty), several slices (192 = 3 x 64), one column block (dk = 16) and eight, on a packed
    batch with tiles of 1, 2, 63 and 64 tokens and an initial state per document."""
    ck, _ = _ops()
    H = 2
    cu = [0, 1, 3, 66, 130, 257]
    T, N = cu[-1], len(cu) - 1
    inp = hp.rounded(po.make_inputs(1, T, H, dk, dv, seed=dk * 3 + dv), torch.bfloat16)
    gen = torch.Generator().manual_seed(5)
    mu0 = torch.randn(N, H, dv, dk, generator=gen) * 0.1
    I0 = 1.0 + torch.rand(N, H, dv, dk, generator=gen)
    o_ref, ov_ref, mu_ref, I_ref = hp.oracle_forward(inp, mu0=mu0, I0=I0, cu=cu, want_var=var)
    d = hp.to_device(inp, gpu_device)
    out, mu, I = _call(ck, d, initial_mu_state=mu0.to(gpu_device), initial_I_state=I0.to(gpu_device),
                       output_final_state=True, output_uncertainty=var, cu_seqlens=torch.tensor(cu, device=gpu_device))
    o, ov = out if var else (out, None)
    assert hp.max_abs(o, o_ref) <= hp.BF16_OUT_ABS_TOL
    if var:
        assert hp.max_abs(ov, ov_ref) <= hp.BF16_OUT_ABS_TOL
    assert hp.max_rel(mu, mu_ref) <= STATE_REL_TOL and hp.max_rel(I, I_ref) <= STATE_REL_TOL
