"""CPU-only checks of the Python boundary: the entry points keep the reference's names, argument
order and defaults; misuse raises what the reference raises; without a GPU the kernels refuse to run
(no silent fallback); palimpsa_ref (the API's plain-PyTorch loop) agrees with the oracle."""
import inspect

import pytest
import torch

from oracle import palimpsa_oracle as po
from palimpsa_amd.ops import palimpsa as ops


def test_exported_names():
    # palimpsa/ops/palimpsa/__init__.py:4-5 of the reference
    for n in ("chunk_palimpsa", "fused_recurrent_palimpsa", "palimpsa_ref"):
        assert callable(getattr(ops, n))
    assert issubclass(ops.ChunkPalimpsa, torch.autograd.Function)
    assert issubclass(ops.FusedRecurrentPalimpsaFunction, torch.autograd.Function)


def _sig(fn):
    return [(p.name, p.default) for p in inspect.signature(fn).parameters.values()]


E = inspect.Parameter.empty


def test_signatures_match_reference():
    # chunk_palimpsa_forgetting_scalar.py:623
    assert _sig(ops.chunk_palimpsa) == [
        ("q", E), ("k", E), ("v", E), ("b", E), ("gt", E), ("g", E), ("Ip", E),
        ("initial_mu_state", None), ("initial_I_state", None), ("scale", None), ("chunk_size", 16),
        ("output_final_state", False), ("output_uncertainty", False), ("cu_seqlens", None)]
    # fused_recurrent_palimpsa.py:258-272
    assert _sig(ops.fused_recurrent_palimpsa) == [
        ("q", E), ("k", E), ("v", E), ("b", E), ("gt", E), ("g", E), ("Ip", E), ("scale", None),
        ("initial_mu_state", None), ("initial_I_state", None), ("output_final_state", False),
        ("output_uncertainty", False), ("cu_seqlens", None)]
    # chunk_palimpsa_forgetting_scalar.py:669
    assert _sig(ops.palimpsa_ref) == [
        ("q", E), ("k", E), ("v", E), ("b", E), ("gt", E), ("g", E), ("Ip", E),
        ("initial_mu_state", None), ("initial_I_state", None), ("scale", None),
        ("output_final_state", False), ("output_uncertainty", False)]
    # autograd Functions: positional order of chunk...py:441 and fused...py:218
    assert [p for p in inspect.signature(ops.ChunkPalimpsa.forward).parameters][1:] == [
        "q", "k", "v", "b", "gt", "g", "Ip", "initial_mu_state", "initial_I_state", "scale", "chunk_size",
        "output_final_state", "output_uncertainty", "cu_seqlens", "chunk_offsets", "int_mu", "int_I"]
    assert [p for p in inspect.signature(ops.FusedRecurrentPalimpsaFunction.forward).parameters][1:] == [
        "q", "k", "v", "b", "gt", "g", "Ip", "scale", "initial_mu_state", "initial_I_state",
        "output_final_state", "output_uncertainty", "cu_seqlens"]


def _inputs(B=2, T=5, H=2, dk=16, dv=16):
    d = po.make_inputs(B, T, H, dk, dv, seed=0)
    return [d[n] for n in ("q", "k", "v", "b", "gt", "g", "Ip")]


def test_varlen_batch_errors_match_reference():
    a = _inputs()
    cu = torch.tensor([0, 5])
    with pytest.raises(ValueError, match="Batch size must be 1"):          # chunk...py:629-630
        ops.chunk_palimpsa(*a, cu_seqlens=cu)
    with pytest.raises(ValueError, match="expected to be 1"):              # fused...py:273-275
        ops.fused_recurrent_palimpsa(*a, cu_seqlens=cu)
    a1 = _inputs(B=1)
    with pytest.raises(ValueError, match="Initial states mismatch"):       # fused...py:276-277
        ops.fused_recurrent_palimpsa(*a1, cu_seqlens=torch.tensor([0, 2, 5]),
                                     initial_mu_state=torch.zeros(3, 2, 16, 16),
                                     initial_I_state=torch.ones(3, 2, 16, 16))
    with pytest.raises(ValueError):
        ops.chunk_palimpsa(*a, chunk_size=0)


def test_cpu_tensors_are_refused_loudly():
    a = _inputs()
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.fused_recurrent_palimpsa(*a)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.chunk_palimpsa(*a)


def test_palimpsa_ref_matches_oracle_and_keeps_the_reference_var_convention():
    q, k, v, b, gt, g, Ip = _inputs(B=2, T=9, H=2, dk=8, dv=6)
    gen = torch.Generator().manual_seed(1)
    mu0 = torch.randn(2, 2, 6, 8, generator=gen)
    I0 = 1.0 + torch.rand(2, 2, 6, 8, generator=gen)
    s = 0.4
    (y, yv), mu, I = ops.palimpsa_ref(q, k, v, b, gt, g, Ip, mu0, I0, scale=s, output_final_state=True,
                                      output_uncertainty=True)
    o, ov2, mu_o, I_o = po.palimpsa_recurrence(q, k, v, b, gt, g, Ip, mu0, I0, scale=s, output_uncertainty=True,
                                               var_scale_power=2)
    assert torch.allclose(y, o, rtol=1e-5, atol=1e-6)
    assert torch.allclose(yv, ov2, rtol=1e-5, atol=1e-6)      # scale**2, chunk...py:709 and :718
    assert torch.allclose(mu, mu_o, rtol=1e-5, atol=1e-6) and torch.allclose(I, I_o, rtol=1e-5)
    # return packing of chunk...py:721-725
    y_only = ops.palimpsa_ref(q, k, v, b, gt, g, Ip)
    assert isinstance(y_only, torch.Tensor) and y_only.shape == (2, 9, 2, 6)
    yb = ops.palimpsa_ref(q.bfloat16(), k.bfloat16(), v.bfloat16(), b.bfloat16(), gt, g, Ip)
    assert yb.dtype == torch.bfloat16


def test_head_dim_padding_rules():
    from palimpsa_amd.ops.palimpsa import _common as cm

    assert [cm.padded_dk(x, True) for x in (1, 16, 31, 33, 65, 100, 130, 200)] == [16, 16, 32, 48, 96, 128, 192, 256]
    assert [cm.padded_dk(x, False) for x in (31, 65, 80)] == [32, 80, 80]
    assert cm.padded_dv(65) == 80
    with pytest.raises(ValueError):
        cm.padded_dk(300, True)


def test_simple_gla_wrappers_keep_the_layer_call_site_keywords():
    """palimpsa/layers/palimpsa.py:296-298 calls q=, k=, v=, g=, initial_state=, output_final_state=, cu_seqlens=."""
    import inspect
    import pytest
    import torch
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla, fused_recurrent_simple_gla
    for fn in (chunk_simple_gla, fused_recurrent_simple_gla):
        names = list(inspect.signature(fn).parameters)
        assert names[:4] == ["q", "k", "v", "g"]
        for n in ("scale", "initial_state", "output_final_state", "cu_seqlens"):
            assert n in names
        x = torch.zeros(1, 4, 2, 16)
        with pytest.raises(ValueError):
            fn(q=x, k=x, v=x, g=None)
        with pytest.raises(ValueError):
            fn(q=x, k=x, v=x, g=torch.zeros(1, 4, 3))


def test_no_cpu_fallback_anywhere():
    """Every entry point of the package refuses CPU tensors instead of computing something on the host."""
    import pytest
    import torch
    from palimpsa_amd.ops.layer_glue import palimpsa_inputs, palimpsa_output_norm
    from palimpsa_amd.ops.palimpsa import DecodeStep
    from palimpsa_amd.ops.simple_gla import SimpleGlaDecodeStep, chunk_simple_gla, fused_recurrent_simple_gla
    x = torch.zeros(1, 4, 2, 16)
    g = torch.zeros(1, 4, 2)
    for fn in (chunk_simple_gla, fused_recurrent_simple_gla):
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            fn(q=x, k=x, v=x, g=g)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        palimpsa_inputs(x, x, x, g, torch.zeros(2), g, x, torch.zeros(2))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        palimpsa_output_norm(x, x, torch.zeros(2), x, torch.ones(16), 1e-6)
    for cls in (DecodeStep, SimpleGlaDecodeStep):
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            cls(1, 2, 16, 16, "cpu")


@pytest.mark.parametrize("cu", [[1, 8], [0, 5, 3, 8], [0, 4, 9], [0, 4, 7], [0]])
def test_cu_seqlens_is_validated_before_anything_runs(cu):
    """cu_seqlens must start at 0, never decrease and end at the token count: the kernels take sequence bounds
    from it, so a malformed array is refused on the host (ValueError) whatever device the tensors are on."""
    from palimpsa_amd.ops.palimpsa import chunk_palimpsa
    from palimpsa_amd.ops.simple_gla import chunk_simple_gla
    H, d, T = 2, 16, 8
    q = torch.zeros(1, T, H, d)
    gt = torch.zeros(1, T, H)
    with pytest.raises(ValueError, match="cu_seqlens"):
        chunk_palimpsa(q, q, q, q, gt, torch.ones(H), torch.ones(H), cu_seqlens=torch.tensor(cu))
    with pytest.raises(ValueError, match="cu_seqlens"):
        chunk_simple_gla(q, q, q, gt, cu_seqlens=torch.tensor(cu))


def test_chunk_table_is_kept_per_cu_seqlens_tensor():
    """The chunk bookkeeping of a packed batch is computed once per cu_seqlens tensor object (every layer of a step
    passes the same one) and recomputed after an in-place change or for another tensor with the same contents."""
    from palimpsa_amd.ops.palimpsa import _common as cm
    cu = torch.tensor([0, 70, 130])
    m1, n1 = cm.chunk_meta(cu, 130, torch.device("cpu"))
    m2, n2 = cm.chunk_meta(cu, 130, torch.device("cpu"))
    assert m1 is m2 and n1 == n2 == 3
    cu[1] = 64                                  # in-place write: the version counter moves
    m3, n3 = cm.chunk_meta(cu, 130, torch.device("cpu"))
    assert m3 is not m1 and n3 == 3 and m3[: 3].tolist() == [0, 1, 3]
    other = torch.tensor([0, 64, 130])
    m4, _ = cm.chunk_meta(other, 130, torch.device("cpu"))
    assert m4 is not m3 and torch.equal(m4, m3)
    with pytest.raises(ValueError):
        cm.chunk_meta(cu, 131, torch.device("cpu"))
    # a host tensor that shares its memory with an array rewritten behind torch's back (no version bump): the entry
    # is compared with the copy taken when it was made
    import numpy as np
    arr = np.array([0, 70, 130], dtype=np.int64)
    shared = torch.from_numpy(arr)
    m5, _ = cm.chunk_meta(shared, 130, torch.device("cpu"))
    arr[1] = 64
    m6, _ = cm.chunk_meta(shared, 130, torch.device("cpu"))
    assert m6 is not m5 and torch.equal(m6, m3)
    arr[2] = 100
    with pytest.raises(ValueError):
        cm.chunk_meta(shared, 130, torch.device("cpu"))
    cm.invalidate_chunk_meta()
    assert cm.chunk_meta(cu, 130, torch.device("cpu"))[0] is not m3
