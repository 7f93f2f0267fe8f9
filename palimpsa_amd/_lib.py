"""ctypes binding of libpalimpsa_hip.so (the C ABI of include/palimpsa_hip.h).

There is no fallback: if the library is missing the import fails with an
instruction to build it, and if a kernel call returns an error it is raised.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libpalimpsa_hip.so")

PAL_ABI_VERSION = 4
PAL_DTYPE_F32, PAL_DTYPE_BF16 = 0, 1
PAL_FLAG_VARLEN, PAL_FLAG_HAS_INIT, PAL_FLAG_STORE_FINAL, PAL_FLAG_HAS_VAR = 1, 2, 4, 8
PAL_FLAG_STATES_TWO_KERNELS, PAL_FLAG_STATES_ONE_PASS, PAL_FLAG_FP32_FAST = 256, 512, 1024
PAL_FLAG_STATE_MU_BF16 = 2048   # pal_recurrent_fwd: mu kept in bf16 between calls (DecodeStep(mu_dtype=torch.bfloat16))
PAL_FLAG_STATES_ONLY = 4096     # pal_chunk_fwd: tile-start states only, outputs untouched
PAL_CHUNK = 64

PAL_E_NULL, PAL_E_DIM, PAL_E_HEADDIM, PAL_E_DTYPE, PAL_E_VARLEN_BATCH = -1, -2, -3, -4, -5
PAL_E_CU_SEQLENS, PAL_E_WORKSPACE, PAL_E_CHUNK, PAL_E_STATE, PAL_E_CAPACITY, PAL_E_ALIGN = -6, -7, -8, -9, -10, -11
PAL_E_SCRATCH = -12
PAL_STATIC_SCRATCH_BYTES = 64 << 20

# dk values the token-serial kernels are compiled for
RECURRENT_DK = (16, 32, 48, 64, 96, 128, 192, 256)


class PalDims(C.Structure):
    _fields_ = [
        ("batch", C.c_int32), ("seq_len", C.c_int32), ("n_seqs", C.c_int32), ("n_heads", C.c_int32),
        ("dk", C.c_int32), ("dv", C.c_int32), ("total_chunks", C.c_int32),
        ("dtype", C.c_int32), ("gate_dtype", C.c_int32), ("var_dtype", C.c_int32),
        ("flags", C.c_uint32), ("scale", C.c_float), ("n_qk_heads", C.c_int32),
    ]


class PalFwdTensors(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in (
        "q", "k", "v", "b", "gt", "g", "Ip", "o", "o_var", "init_mu", "init_I", "final_mu", "final_I",
        "cu_seqlens", "chunk_table", "chunk_offsets", "chunk_mu", "chunk_I")]


class PalBwdTensors(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in (
        "d_o", "d_o_var", "dq", "dk", "dv", "db", "dgt", "dg", "dIp", "d_init_mu", "d_init_I")]


class PalGlueDims(C.Structure):
    _fields_ = ([(n, C.c_int32) for n in ("tokens", "n_heads", "n_qk_heads", "dk", "dv", "dtype")] +
                [("eps", C.c_float), ("dt_min", C.c_float), ("dt_max", C.c_float), ("norm_over_heads", C.c_int32)])


class PalPrologueTensors(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in (
        "q_raw", "k_raw", "x", "dt_raw", "bs_raw", "b_raw", "dt_bias", "b_scale", "q", "k", "v", "b", "gt")]


class PalPrologueGrads(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in (
        "dq", "dk", "dv", "db", "dgt", "dq_raw", "dk_raw", "dx", "db_raw", "ddt_raw", "dbs_raw", "ddt_bias", "db_scale")]


class PalEpilogueTensors(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("o", "x", "D", "gate", "weight", "y", "rstd")]


class PalEpilogueGrads(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("dy", "d_o", "dx", "dgate", "dD", "dweight")]


class PalimpsaHipError(RuntimeError):
    def __init__(self, code: int, where: str, text: str):
        super().__init__(f"{where} failed with code {code}: {text}")
        self.code = code


_lib: Optional[C.CDLL] = None


def load() -> C.CDLL:
    """Load the shared library once; raises ImportError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: build it with `python -m palimpsa_amd.build` "
            "(needs hipcc; the kernels target gfx950). There is no CPU or eager fallback.")
    lib = C.CDLL(LIB_PATH)
    P = C.POINTER
    lib.pal_abi_version.restype = C.c_int
    lib.pal_abi_version.argtypes = []
    lib.pal_strerror.restype = C.c_char_p
    lib.pal_strerror.argtypes = [C.c_int]
    lib.pal_validate_dims.restype = C.c_int
    lib.pal_validate_dims.argtypes = [P(PalDims)]
    lib.pal_build_chunk_table.restype = C.c_int
    lib.pal_build_chunk_table.argtypes = [P(C.c_int64), C.c_int32, P(C.c_int32), C.c_int32, P(C.c_int32)]
    for name in ("pal_recurrent_fwd", "pal_chunk_fwd", "pal_chunk_fwd_static", "pal_gla_chunk_fwd",
                 "pal_gla_recurrent_fwd"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [P(PalDims), P(PalFwdTensors), C.c_void_p]
    for name in ("pal_recurrent_bwd", "pal_chunk_bwd", "pal_gla_chunk_bwd"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [P(PalDims), P(PalFwdTensors), P(PalBwdTensors), C.c_void_p, C.c_size_t, C.c_void_p]
    for name in ("pal_recurrent_bwd_workspace_bytes", "pal_chunk_bwd_workspace_bytes",
                 "pal_gla_chunk_bwd_workspace_bytes"):
        fn = getattr(lib, name)
        fn.restype = C.c_size_t
        fn.argtypes = [P(PalDims)]
    lib.pal_prologue_fwd.restype = C.c_int
    lib.pal_prologue_fwd.argtypes = [P(PalGlueDims), P(PalPrologueTensors), C.c_void_p]
    lib.pal_prologue_bwd.restype = C.c_int
    lib.pal_prologue_bwd.argtypes = [P(PalGlueDims), P(PalPrologueTensors), P(PalPrologueGrads), C.c_void_p, C.c_size_t,
                                     C.c_void_p]
    lib.pal_epilogue_fwd.restype = C.c_int
    lib.pal_epilogue_fwd.argtypes = [P(PalGlueDims), P(PalEpilogueTensors), C.c_void_p]
    lib.pal_epilogue_bwd.restype = C.c_int
    lib.pal_epilogue_bwd.argtypes = [P(PalGlueDims), P(PalEpilogueTensors), P(PalEpilogueGrads), C.c_void_p, C.c_size_t,
                                     C.c_void_p]
    for name in ("pal_prologue_bwd_workspace_bytes", "pal_epilogue_bwd_workspace_bytes"):
        fn = getattr(lib, name)
        fn.restype = C.c_size_t
        fn.argtypes = [P(PalGlueDims)]
    lib.pal_state_pass_applies.restype = C.c_int
    lib.pal_state_pass_applies.argtypes = [P(PalDims), C.c_int]
    lib.pal_chunk_bwd_supported.restype = C.c_int
    lib.pal_chunk_bwd_supported.argtypes = [C.c_int32, C.c_int32, C.c_int32, C.c_uint32]
    lib.pal_profile_enable.restype = C.c_int
    lib.pal_profile_enable.argtypes = [C.c_int]
    lib.pal_profile_kernel_count.restype = C.c_int
    lib.pal_profile_kernel_count.argtypes = []
    lib.pal_profile_kernel_name.restype = C.c_char_p
    lib.pal_profile_kernel_name.argtypes = [C.c_int]
    lib.pal_profile_read.restype = C.c_int
    lib.pal_profile_read.argtypes = [C.c_int, P(C.c_double), P(C.c_int64)]
    if lib.pal_abi_version() != PAL_ABI_VERSION:
        raise ImportError(f"{LIB_PATH}: ABI version {lib.pal_abi_version()} != expected {PAL_ABI_VERSION}; rebuild")
    _lib = lib
    return lib


# How the chunked entry points build the tile-start states (PAL_FLAG_STATES_* of the C ABI): 0 = chosen by shape,
# 1 = two kernels, 2 = one pass wherever it applies.  A knob of this Python layer for tests and measurements (the
# library itself keeps no such state); initial value from the environment variable PALIMPSA_STATE_PASS_MODE.
_state_pass_mode = int(os.environ.get("PALIMPSA_STATE_PASS_MODE", "0"))


def set_state_pass_mode(mode: int) -> None:
    global _state_pass_mode
    if mode not in (0, 1, 2):
        raise ValueError(f"state pass mode must be 0, 1 or 2, got {mode!r}")
    _state_pass_mode = mode


# fp32 rows through the chunked entry points: False (default) = operands split into two bf16 halves, results within
# 1e-4 of the fp32 recurrence; True = single bf16/f16 operands as for bf16 rows (PAL_FLAG_FP32_FAST; about twice as
# fast, errors of 1e-3 .. 1e-2).  Initial value from the environment variable PALIMPSA_FP32_FAST.
_fp32_fast = os.environ.get("PALIMPSA_FP32_FAST", "0") not in ("", "0")


def set_fp32_fast(on: bool) -> None:
    global _fp32_fast
    _fp32_fast = bool(on)


# Backward of the token-serial entry point: sequences of at least this many tokens on average are handed to the
# chunked backward kernels (tile-start states from a states-only forward, then pal_chunk_bwd; fp32 rows keep the fp32
# bar there through split operands), shorter ones run the token-serial backward kernel, which walks a sequence
# token by token (measured at 196608 token-heads of 64 x 64, fp32 rows: 256 sequences of 64 tokens 4.97 ms token-serial
# against 2.9 ms chunked, 8 sequences of 2048 tokens 7.05 against 2.93; a tile costs the same however few of its 64
# tokens are real, so below a tile per sequence the token-serial kernel wins).  None = never.  Initial value from the environment variable PALIMPSA_RECURRENT_BWD_CHUNK_MIN.
_recurrent_bwd_chunk_min = os.environ.get("PALIMPSA_RECURRENT_BWD_CHUNK_MIN", "64")
_recurrent_bwd_chunk_min = None if _recurrent_bwd_chunk_min in ("", "none", "None") else int(_recurrent_bwd_chunk_min)


def set_recurrent_bwd_chunk_min(tokens) -> None:
    global _recurrent_bwd_chunk_min
    _recurrent_bwd_chunk_min = None if tokens is None else int(tokens)


def recurrent_bwd_chunk_min():
    return _recurrent_bwd_chunk_min


def state_pass_flags() -> int:
    """The PalDims.flags bits this Python layer adds to every call of a chunked entry point."""
    return (0, PAL_FLAG_STATES_TWO_KERNELS, PAL_FLAG_STATES_ONE_PASS)[_state_pass_mode] | \
        (PAL_FLAG_FP32_FAST if _fp32_fast else 0)


def strerror(code: int) -> str:
    return load().pal_strerror(int(code)).decode()


def check(code: int, where: str) -> None:
    """Map a pal_* return code to the Python exception the reference would raise."""
    if code == 0:
        return
    text = strerror(code)
    if code in (PAL_E_VARLEN_BATCH, PAL_E_CU_SEQLENS, PAL_E_HEADDIM, PAL_E_DIM, PAL_E_DTYPE, PAL_E_STATE, PAL_E_SCRATCH):
        raise ValueError(f"{where}: {text} (code {code})")
    raise PalimpsaHipError(code, where, text)


def build_chunk_table(cu_seqlens_host):
    """Host chunk bookkeeping for packed batches: returns (table int32 [n,4], offsets int32 [N+1])."""
    import numpy as np

    lib = load()
    cu = np.ascontiguousarray(np.asarray(cu_seqlens_host, dtype=np.int64))
    n_seqs = int(cu.shape[0]) - 1
    cu_p = cu.ctypes.data_as(C.POINTER(C.c_int64))
    total = lib.pal_build_chunk_table(cu_p, n_seqs, None, 0, None)
    if total < 0:
        check(total, "pal_build_chunk_table")
    table = np.zeros((max(total, 1), 4), dtype=np.int32)
    offsets = np.zeros((n_seqs + 1,), dtype=np.int32)
    rc = lib.pal_build_chunk_table(cu_p, n_seqs, table.ctypes.data_as(C.POINTER(C.c_int32)), int(table.shape[0]),
                                   offsets.ctypes.data_as(C.POINTER(C.c_int32)))
    if rc < 0:
        check(rc, "pal_build_chunk_table")
    return table[:total], offsets


def profile_enable(on: bool) -> None:
    """Switch the library's per-kernel HIP-event timing on or off (resets the counters)."""
    load().pal_profile_enable(1 if on else 0)


def profile_read():
    """{kernel name: (total_ms, launches)} for every kernel launched since profile_enable(True)."""
    lib = load()
    out = {}
    for i in range(lib.pal_profile_kernel_count()):
        ms, n = C.c_double(0.0), C.c_int64(0)
        lib.pal_profile_read(i, C.byref(ms), C.byref(n))
        if n.value:
            out[lib.pal_profile_kernel_name(i).decode()] = (ms.value, n.value)
    return out
