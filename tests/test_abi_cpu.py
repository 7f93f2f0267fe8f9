"""CPU-only checks of the C-ABI shared library: it loads, exports every symbol the header declares,
rejects bad arguments before any HIP call, and the host-side chunk bookkeeping matches the oracle.
No kernel is launched here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from oracle import palimpsa_oracle as po

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "palimpsa_hip.h")


@pytest.fixture(scope="module")
def L():
    from palimpsa_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        from palimpsa_amd import build

        build.build()
    _lib.load()
    return _lib


def _declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(pal_[a-z_0-9]+)\s*\(", src)))


def test_library_exports_every_declared_symbol(L):
    lib = L.load()
    names = _declared_functions()
    assert {"pal_recurrent_fwd", "pal_recurrent_bwd", "pal_chunk_fwd", "pal_chunk_bwd", "pal_build_chunk_table",
            "pal_strerror", "pal_abi_version", "pal_validate_dims"} <= set(names)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in palimpsa_hip.h but not exported"


def test_abi_version_and_strerror(L):
    lib = L.load()
    assert lib.pal_abi_version() == L.PAL_ABI_VERSION
    assert L.strerror(0) == "ok"
    for code in range(-11, 0):
        assert "unknown" not in L.strerror(code)
    assert "unknown" in L.strerror(-99)


def _dims(L, **kw):
    d = dict(batch=2, seq_len=16, n_seqs=2, n_heads=2, dk=32, dv=32, total_chunks=2, dtype=L.PAL_DTYPE_BF16,
             gate_dtype=L.PAL_DTYPE_F32, var_dtype=L.PAL_DTYPE_F32, flags=0, scale=1.0)
    d.update(kw)
    return L.PalDims(**d)


def test_validate_dims_codes(L):
    v = L.load().pal_validate_dims
    assert v(_dims(L)) == 0
    assert v(None) == L.PAL_E_NULL
    assert v(_dims(L, batch=0)) == L.PAL_E_DIM
    assert v(_dims(L, seq_len=-1)) == L.PAL_E_DIM
    assert v(_dims(L, n_heads=0)) == L.PAL_E_DIM
    assert v(_dims(L, dk=31)) == L.PAL_E_HEADDIM
    assert v(_dims(L, dv=272)) == L.PAL_E_HEADDIM
    assert v(_dims(L, dk=8)) == L.PAL_E_HEADDIM
    assert v(_dims(L, dtype=7)) == L.PAL_E_DTYPE
    assert v(_dims(L, gate_dtype=-1)) == L.PAL_E_DTYPE
    assert v(_dims(L, flags=L.PAL_FLAG_VARLEN)) == L.PAL_E_VARLEN_BATCH      # B != 1 with cu_seqlens
    assert v(_dims(L, n_seqs=3)) == L.PAL_E_DIM                               # fixed length: N must equal B
    assert v(_dims(L, batch=1, n_seqs=40, flags=L.PAL_FLAG_VARLEN)) == L.PAL_E_CU_SEQLENS  # more docs than tokens
    assert v(_dims(L, scale=float("nan"))) == L.PAL_E_DIM
    assert v(_dims(L, batch=1, n_seqs=3, flags=L.PAL_FLAG_VARLEN)) == 0


def _fake(addr=0x1000):
    return C.c_void_p(addr)


def _fwd_tensors(L, **kw):
    names = ("q", "k", "v", "b", "gt", "g", "Ip", "o")
    t = {n: _fake(0x1000 * (i + 1)) for i, n in enumerate(names)}
    t.update(kw)
    return L.PalFwdTensors(**t)


def test_entry_points_reject_bad_arguments_without_touching_a_gpu(L):
    """Every error below is detected by the host-side checks, so no HIP call is made (this test runs
    on machines without a GPU; the pointers are fake and never dereferenced)."""
    lib = L.load()
    assert lib.pal_recurrent_fwd(None, None, None) == L.PAL_E_NULL
    assert lib.pal_recurrent_fwd(_dims(L), None, None) == L.PAL_E_NULL
    assert lib.pal_recurrent_fwd(_dims(L), _fwd_tensors(L, q=None), None) == L.PAL_E_NULL
    assert lib.pal_recurrent_fwd(_dims(L, dk=24), _fwd_tensors(L), None) == L.PAL_E_HEADDIM
    assert lib.pal_recurrent_fwd(_dims(L, dk=80), _fwd_tensors(L), None) == L.PAL_E_HEADDIM   # chunk-only size
    assert lib.pal_recurrent_fwd(_dims(L), _fwd_tensors(L, q=_fake(0x1004)), None) == L.PAL_E_ALIGN
    # a gate is fetched as the aligned 32-bit word that holds it: a bf16 gate tensor on a 2-byte boundary is refused
    assert lib.pal_recurrent_fwd(_dims(L, gate_dtype=L.PAL_DTYPE_BF16), _fwd_tensors(L, gt=_fake(0x5002)),
                                 None) == L.PAL_E_ALIGN
    assert lib.pal_recurrent_fwd(_dims(L), _fwd_tensors(L, gt=_fake(0x5002)), None) == L.PAL_E_ALIGN
    # state flags and pointers must agree
    assert lib.pal_recurrent_fwd(_dims(L, flags=L.PAL_FLAG_HAS_INIT), _fwd_tensors(L), None) == L.PAL_E_STATE
    assert lib.pal_recurrent_fwd(_dims(L), _fwd_tensors(L, init_mu=_fake(), init_I=_fake()), None) == L.PAL_E_STATE
    assert lib.pal_recurrent_fwd(_dims(L, flags=L.PAL_FLAG_STORE_FINAL), _fwd_tensors(L, final_mu=_fake()),
                                 None) == L.PAL_E_STATE
    assert lib.pal_recurrent_fwd(_dims(L, flags=L.PAL_FLAG_HAS_VAR), _fwd_tensors(L), None) == L.PAL_E_NULL
    # varlen flag without cu_seqlens, and the other way round
    assert lib.pal_recurrent_fwd(_dims(L, batch=1, n_seqs=2, flags=L.PAL_FLAG_VARLEN), _fwd_tensors(L),
                                 None) == L.PAL_E_CU_SEQLENS
    assert lib.pal_recurrent_fwd(_dims(L), _fwd_tensors(L, cu_seqlens=_fake()), None) == L.PAL_E_CU_SEQLENS
    # chunk path
    assert lib.pal_chunk_fwd(_dims(L, flags=L.PAL_FLAG_STORE_FINAL), _fwd_tensors(L, final_mu=_fake(), final_I=_fake()),
                             None) == L.PAL_E_NULL                               # chunk_mu / chunk_I missing
    ok_chunk = dict(final_mu=_fake(), final_I=_fake(), chunk_mu=_fake(0x9000), chunk_I=_fake(0xa000))
    assert lib.pal_chunk_fwd(_dims(L, flags=L.PAL_FLAG_STORE_FINAL, total_chunks=5), _fwd_tensors(L, **ok_chunk),
                             None) == L.PAL_E_CHUNK                              # 2 sequences of 16 tokens = 2 tiles
    assert lib.pal_chunk_bwd(_dims(L), _fwd_tensors(L, chunk_mu=_fake(0x9000), chunk_I=_fake(0xa000)), None, None, 0,
                             None) == L.PAL_E_NULL
    gr = L.PalBwdTensors(**{n: _fake(0x1000 * (i + 20)) for i, n in enumerate(
        ("d_o", "dq", "dk", "dv", "db", "dgt", "dg", "dIp"))})
    assert lib.pal_chunk_bwd(_dims(L), _fwd_tensors(L, chunk_mu=_fake(0x9000), chunk_I=_fake(0xa000)), gr, None, 0,
                             None) == L.PAL_E_WORKSPACE
    assert lib.pal_chunk_bwd_workspace_bytes(_dims(L)) > 0
    assert lib.pal_chunk_bwd_workspace_bytes(_dims(L, dk=5)) == 0
    # the bf16 cache format of the mean state belongs to pal_recurrent_fwd alone
    mu16 = L.PAL_FLAG_STATE_MU_BF16
    assert lib.pal_chunk_fwd(_dims(L, flags=L.PAL_FLAG_STORE_FINAL | mu16, total_chunks=2), _fwd_tensors(L, **ok_chunk),
                             None) == L.PAL_E_STATE
    assert lib.pal_chunk_bwd(_dims(L, flags=mu16), _fwd_tensors(L, chunk_mu=_fake(0x9000), chunk_I=_fake(0xa000)), gr,
                             None, 0, None) == L.PAL_E_STATE
    assert lib.pal_recurrent_fwd(_dims(L, flags=mu16 | L.PAL_FLAG_HAS_INIT), _fwd_tensors(L), None) == L.PAL_E_STATE


def test_error_codes_map_to_python_exceptions(L):
    with pytest.raises(ValueError):
        L.check(L.PAL_E_VARLEN_BATCH, "x")
    with pytest.raises(ValueError):
        L.check(L.PAL_E_HEADDIM, "x")
    with pytest.raises(L.PalimpsaHipError):
        L.check(L.PAL_E_WORKSPACE, "x")
    with pytest.raises(L.PalimpsaHipError):
        L.check(1, "x")          # a hipError_t
    L.check(0, "x")


def test_chunk_table_matches_oracle(L):
    rng = np.random.RandomState(0)
    for _ in range(20):
        lens = rng.randint(0, 300, size=rng.randint(1, 9))
        lens[rng.randint(len(lens))] += 1            # at least one token overall
        cu = np.concatenate([[0], np.cumsum(lens)])
        table, offsets = L.build_chunk_table(cu)
        ref = po.build_chunk_table(cu.tolist(), 64)
        assert [tuple(r[:3]) for r in table.tolist()] == ref
        assert offsets.tolist() == po.chunk_offsets(cu.tolist(), 64)
        # index inside the sequence restarts at every document
        for row in table.tolist():
            assert row[1] == cu[row[0]] + 64 * row[3]
    cu = po.make_varlen_lengths(32768, seed=0)
    table, offsets = L.build_chunk_table(cu)
    assert table[:, 2].sum() == 32768 and table[:, 2].max() <= 64 and table[:, 2].min() >= 1


def test_chunk_table_rejects_bad_cu_seqlens(L):
    with pytest.raises(ValueError):
        L.build_chunk_table([1, 5])            # does not start at 0
    with pytest.raises(ValueError):
        L.build_chunk_table([0, 9, 5])         # decreasing
    lib = L.load()
    cu = (C.c_int64 * 3)(0, 100, 200)
    out = (C.c_int32 * 8)()
    assert lib.pal_build_chunk_table(cu, 2, out, 2, None) == L.PAL_E_CAPACITY
    assert lib.pal_build_chunk_table(None, 2, None, 0, None) == L.PAL_E_NULL


def test_states_only_forward_checks_its_arguments(L):
    """PAL_FLAG_STATES_ONLY: pal_chunk_fwd fills the tile-start states and leaves the outputs alone, so o may be NULL;
    everything else is checked as usual, before any HIP call."""
    lib = L.load()
    so = L.PAL_FLAG_STATES_ONLY
    assert lib.pal_chunk_fwd(_dims(L, flags=so), _fwd_tensors(L, o=None), None) == L.PAL_E_NULL             # no state buffers
    assert lib.pal_chunk_fwd(_dims(L, flags=so, total_chunks=3),
                             _fwd_tensors(L, o=None, chunk_mu=_fake(0x9000), chunk_I=_fake(0xa000)), None) == L.PAL_E_CHUNK
    assert lib.pal_chunk_fwd(_dims(L, flags=so), _fwd_tensors(L, o=None, q=None, chunk_mu=_fake(0x9000), chunk_I=_fake(0xa000)),
                             None) == L.PAL_E_NULL
    assert lib.pal_chunk_fwd(_dims(L, flags=so | L.PAL_FLAG_HAS_INIT),
                             _fwd_tensors(L, o=None, chunk_mu=_fake(0x9000), chunk_I=_fake(0xa000)), None) == L.PAL_E_STATE


def test_simple_gla_entry_points_reject_bad_arguments(L):
    """Host-side checks of the entry points without the precision state (no HIP call before they pass)."""
    lib = L.load()
    ok = dict(chunk_mu=_fake(0x9000), chunk_I=_fake(0xa000))
    for fn in (lib.pal_gla_chunk_fwd, lib.pal_gla_recurrent_fwd):
        assert fn(None, None, None) == L.PAL_E_NULL
        assert fn(_dims(L), None, None) == L.PAL_E_NULL
        assert fn(_dims(L), _fwd_tensors(L, q=None, **ok), None) == L.PAL_E_NULL
        assert fn(_dims(L, dv=40), _fwd_tensors(L, **ok), None) == L.PAL_E_HEADDIM
        assert fn(_dims(L, flags=L.PAL_FLAG_HAS_VAR), _fwd_tensors(L, o_var=_fake(), **ok), None) == L.PAL_E_STATE
        assert fn(_dims(L, flags=L.PAL_FLAG_HAS_INIT), _fwd_tensors(L, **ok), None) == L.PAL_E_STATE
        assert fn(_dims(L), _fwd_tensors(L, final_mu=_fake(), **ok), None) == L.PAL_E_STATE
        assert fn(_dims(L), _fwd_tensors(L, cu_seqlens=_fake(), **ok), None) == L.PAL_E_CU_SEQLENS
        assert fn(_dims(L), _fwd_tensors(L, v=_fake(0x3008), **ok), None) == L.PAL_E_ALIGN
        assert fn(_dims(L, gate_dtype=L.PAL_DTYPE_BF16), _fwd_tensors(L, gt=_fake(0x5002), **ok), None) == L.PAL_E_ALIGN
    # q, k with fewer heads than v: a divisor of the head count, as for the Palimpsa entry points
    assert lib.pal_gla_chunk_fwd(_dims(L, n_qk_heads=3), _fwd_tensors(L, **ok), None) == L.PAL_E_DIM
    # the chunked form needs both tile buffers and a consistent tile count
    assert lib.pal_gla_chunk_fwd(_dims(L), _fwd_tensors(L, chunk_mu=_fake(0x9000)), None) == L.PAL_E_NULL
    assert lib.pal_gla_chunk_fwd(_dims(L), _fwd_tensors(L, chunk_I=_fake(0xa000)), None) == L.PAL_E_NULL
    assert lib.pal_gla_chunk_fwd(_dims(L, total_chunks=3), _fwd_tensors(L, **ok), None) == L.PAL_E_CHUNK
    assert lib.pal_gla_chunk_fwd(_dims(L, batch=1, n_seqs=2, seq_len=32, flags=L.PAL_FLAG_VARLEN),
                                 _fwd_tensors(L, cu_seqlens=_fake(), **ok), None) == L.PAL_E_NULL      # chunk tables
    # backward
    gr = L.PalBwdTensors(**{n: _fake(0x1000 * (i + 20)) for i, n in enumerate(("d_o", "dq", "dk", "dv", "dgt", "dg"))})
    assert lib.pal_gla_chunk_bwd(_dims(L), _fwd_tensors(L, **ok), None, None, 0, None) == L.PAL_E_NULL
    assert lib.pal_gla_chunk_bwd(_dims(L), _fwd_tensors(L, **ok), gr, None, 0, None) == L.PAL_E_WORKSPACE
    need = lib.pal_gla_chunk_bwd_workspace_bytes(_dims(L))
    # D (fp32) and G (bf16) tiles, two rows of dot products, per-sequence shares of dg
    assert need >= 2 * 2 * 32 * 32 * (4 + 2) + 2 * 2 * 16 * 2 * 4 + 2 * 2 * 4
    assert lib.pal_gla_chunk_bwd(_dims(L), _fwd_tensors(L, **ok), gr, _fake(0x100000), need - 1, None) == L.PAL_E_WORKSPACE
    gr2 = L.PalBwdTensors(**{n: _fake(0x1000 * (i + 20)) for i, n in enumerate(("d_o", "dq", "dk", "dv", "dgt", "dg", "d_init_mu"))})
    assert lib.pal_gla_chunk_bwd(_dims(L), _fwd_tensors(L, **ok), gr2, _fake(0x100000), need, None) == L.PAL_E_STATE
    assert lib.pal_gla_chunk_bwd_workspace_bytes(_dims(L, dk=5)) == 0


def test_layer_glue_entry_points_reject_bad_arguments(L):
    lib = L.load()

    def gd(**kw):
        d = dict(tokens=10, n_heads=4, n_qk_heads=2, dk=32, dv=64, dtype=L.PAL_DTYPE_BF16, eps=1e-6)
        d.update(kw)
        return L.PalGlueDims(**d)

    names = ("q_raw", "k_raw", "x", "dt_raw", "bs_raw", "b_raw", "dt_bias", "b_scale", "q", "k", "v", "b", "gt")

    def pt(**kw):
        t = {n: _fake(0x1000 * (i + 1)) for i, n in enumerate(names)}
        t.update(kw)
        return L.PalPrologueTensors(**t)

    assert lib.pal_prologue_fwd(None, None, None) == L.PAL_E_NULL
    assert lib.pal_prologue_fwd(gd(), None, None) == L.PAL_E_NULL
    assert lib.pal_prologue_fwd(gd(tokens=0), pt(), None) == L.PAL_E_DIM
    assert lib.pal_prologue_fwd(gd(n_qk_heads=3), pt(), None) == L.PAL_E_DIM           # 4 heads not a multiple of 3
    assert lib.pal_prologue_fwd(gd(dk=12), pt(), None) == L.PAL_E_HEADDIM
    assert lib.pal_prologue_fwd(gd(dv=264), pt(), None) == L.PAL_E_HEADDIM
    assert lib.pal_prologue_fwd(gd(dtype=7), pt(), None) == L.PAL_E_DTYPE
    assert lib.pal_prologue_fwd(gd(), pt(x=None), None) == L.PAL_E_NULL
    assert lib.pal_prologue_fwd(gd(), pt(b=None), None) == L.PAL_E_STATE                # b_raw without b
    assert lib.pal_prologue_fwd(gd(), pt(b_scale=None), None) == L.PAL_E_NULL
    assert lib.pal_prologue_fwd(gd(), pt(q=_fake(0x9004)), None) == L.PAL_E_ALIGN
    assert lib.pal_prologue_bwd(gd(), pt(), None, None, 0, None) == L.PAL_E_NULL
    gnames = ("dq", "dk", "dv", "db", "dgt", "dq_raw", "dk_raw", "dx", "db_raw", "ddt_raw", "dbs_raw", "ddt_bias", "db_scale")
    gr = L.PalPrologueGrads(**{n: _fake(0x1000 * (i + 30)) for i, n in enumerate(gnames)})
    assert lib.pal_prologue_bwd(gd(), pt(), gr, None, 0, None) == L.PAL_E_WORKSPACE
    assert lib.pal_prologue_bwd_workspace_bytes(gd()) > 0 and lib.pal_prologue_bwd_workspace_bytes(gd(dk=3)) == 0

    def et(**kw):
        t = {n: _fake(0x1000 * (i + 1)) for i, n in enumerate(("o", "x", "D", "gate", "weight", "y", "rstd"))}
        t.update(kw)
        return L.PalEpilogueTensors(**t)

    assert lib.pal_epilogue_fwd(gd(), None, None) == L.PAL_E_NULL
    assert lib.pal_epilogue_fwd(gd(), et(weight=None), None) == L.PAL_E_NULL
    assert lib.pal_epilogue_fwd(gd(), et(D=None), None) == L.PAL_E_NULL                  # x without D
    assert lib.pal_epilogue_fwd(gd(), et(o=_fake(0x1008)), None) == L.PAL_E_ALIGN
    eg = L.PalEpilogueGrads(**{n: _fake(0x1000 * (i + 40)) for i, n in enumerate(("dy", "d_o", "dx", "dgate", "dD", "dweight"))})
    assert lib.pal_epilogue_bwd(gd(), et(), None, None, 0, None) == L.PAL_E_NULL
    assert lib.pal_epilogue_bwd(gd(), et(), L.PalEpilogueGrads(dy=_fake(), d_o=_fake(0x2000), dweight=_fake(0x3000)), None, 0,
                                None) == L.PAL_E_NULL                                    # dx / dD / dgate missing
    assert lib.pal_epilogue_bwd(gd(), et(), eg, None, 0, None) == L.PAL_E_WORKSPACE
    assert lib.pal_epilogue_bwd_workspace_bytes(gd()) > 0

    # the MetaMamba2 layer's form: no bs_raw (the multiplier is the clamped time step), q/k rows all present or all absent
    mamba = dict(bs_raw=None, q_raw=None, k_raw=None, q=None, k=None)
    assert lib.pal_prologue_fwd(gd(dt_min=0.5, dt_max=0.1), pt(**mamba), None) == L.PAL_E_DIM      # bounds out of order
    assert lib.pal_prologue_fwd(gd(dt_min=float("nan")), pt(**mamba), None) == L.PAL_E_DIM
    assert lib.pal_prologue_fwd(gd(), pt(**dict(mamba, k=_fake(0x7000))), None) == L.PAL_E_NULL    # one of the four q/k tensors
    assert lib.pal_prologue_fwd(gd(), pt(q_raw=None, k_raw=None, q=None, k=None), None) == L.PAL_E_NULL   # bs_raw needs q, k
    assert lib.pal_prologue_fwd(gd(), pt(**dict(mamba, gt=None)), None) == L.PAL_E_NULL
    gm = L.PalPrologueGrads(**{n: _fake(0x1000 * (i + 30)) for i, n in enumerate(gnames)
                               if n not in ("dq", "dk", "dq_raw", "dk_raw", "dbs_raw")})
    assert lib.pal_prologue_bwd(gd(dt_max=1.0), pt(**mamba), gm, None, 0, None) == L.PAL_E_WORKSPACE   # arguments accepted
    assert lib.pal_prologue_bwd(gd(), pt(), gm, None, 0, None) == L.PAL_E_NULL                     # the layer form needs them
    # norm over all heads of a token: up to 4096 entries
    assert lib.pal_epilogue_fwd(gd(norm_over_heads=1, n_heads=32, n_qk_heads=32, dv=256), et(), None) == L.PAL_E_DIM
    assert lib.pal_epilogue_bwd(gd(norm_over_heads=1), et(), eg, None, 0, None) == L.PAL_E_WORKSPACE
    assert lib.pal_epilogue_bwd_workspace_bytes(gd(norm_over_heads=1, tokens=1600)) == 100 * 4 * (256 + 32)   # one row per 16 tokens


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    """Without the built library the package raises ImportError with the build instruction; nothing is computed."""
    from palimpsa_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libpalimpsa_hip.so"))
    with pytest.raises(ImportError, match="palimpsa_amd.build"):
        _lib.load()
