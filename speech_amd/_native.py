"""ctypes binding of libmi_transducer.so (the HIP kernels behind a plain C ABI).

The library is built in-tree by `build()` (hipcc, gfx950) and loaded from
speech_amd/csrc/.  There is no fallback: if the library cannot be loaded, every
entry point raises, so a silent non-HIP path cannot exist.
"""

import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.join(_HERE, "csrc")
INCLUDE_DIR = os.path.join(os.path.dirname(_HERE), "include")
# MI_TRANSDUCER_LIB lets a kernel developer point at an experimental build of the same ABI
LIB_PATH = os.environ.get("MI_TRANSDUCER_LIB") or os.path.join(CSRC_DIR, "libmi_transducer.so")
SOURCES = [os.path.join(CSRC_DIR, "mi_transducer.hip")]
# the host (CPU) implementation of the RNNT loss: plain C++ / OpenMP, its own library and header
CPU_LIB_PATH = os.path.join(CSRC_DIR, "libmi_transducer_cpu.so")
CPU_SOURCES = [os.path.join(CSRC_DIR, "mi_cpu.cpp")]
CPU_ABI_VERSION = 1
CXX_FLAGS = ["-O3", "-std=c++17", "-fPIC", "-shared", "-fopenmp", "-Wall", "-Wextra"]

ABI_VERSION = 20
SUCCESS, INVALID_VALUE, LAUNCH_FAILURE, TOO_LARGE = 0, 1, 2, 3
STATIC_WORKSPACE_BYTES = 64 << 20
DTYPE_F32, DTYPE_BF16, DTYPE_F16 = 0, 1, 2
RIDERS_AUTO, RIDERS_OFF, RIDERS_ON = -1, 0, 1  # `riders` of the combined mi_*_loss entry points

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # keep the compiler from forming packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the first dwords of a kernel's arguments arrive in scalar registers with the wave instead of being fetched by
    # its first instructions (the kernels order their arguments for it)
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]  # fmt: skip


def _compile(cmd, what, verbose):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or proc.returncode != 0:
        print(" ".join(cmd))
        print(proc.stdout)
        print(proc.stderr)
    if proc.returncode != 0:
        raise RuntimeError(f"building {what} failed:\n" + proc.stderr)


def build(verbose=False):
    """Compile the HIP sources into speech_amd/csrc/libmi_transducer.so (cross-compiles without a GPU) and the host
    implementation of the RNNT loss into speech_amd/csrc/libmi_transducer_cpu.so."""
    hipcc = os.environ.get("HIPCC", "hipcc")
    _compile([hipcc, *HIPCC_FLAGS, "-I", INCLUDE_DIR, "-o", LIB_PATH, *SOURCES], "libmi_transducer.so", verbose)
    build_cpu(verbose)
    global _lib
    _lib = None
    return LIB_PATH


def build_cpu(verbose=False):
    cxx = os.environ.get("CXX", "g++")
    _compile([cxx, *CXX_FLAGS, "-I", INCLUDE_DIR, "-o", CPU_LIB_PATH, *CPU_SOURCES], "libmi_transducer_cpu.so", verbose)
    global _cpu_lib
    _cpu_lib = None
    return CPU_LIB_PATH


_lib = None

_c_int, _c_float, _c_size_t, _vp = ctypes.c_int, ctypes.c_float, ctypes.c_size_t, ctypes.c_void_p

# name -> argtypes, in the order of include/mi_transducer.h
_SIGNATURES = {
    "mi_transducer_abi_version": [],
    "mi_transducer_workspace_bytes": [_c_int, _c_int, _c_int, _c_int, ctypes.POINTER(_c_size_t)],
    "mi_rnnt_forward": [_vp, _c_int, _vp, _vp, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int,
                        _vp, _vp, _c_size_t, _vp],
    "mi_rnnt_backward": [_vp, _c_int, _vp, _vp, _vp, _vp, _vp, _c_int, _c_float, _c_int, _c_int, _c_int, _c_int,
                         _c_int, _c_int, _c_float, _c_float, _vp, _c_size_t, _vp],
    "mi_rnnt_loss": [_vp, _c_int, _vp, _vp, _vp, _vp, _vp, _vp, _c_int, _c_float, _c_int, _c_int, _c_int, _c_int,
                     _c_int, _c_float, _c_float, _c_int, _vp, _c_size_t, _vp],
    "mi_transducer_init": [],
    "mi_rnnt_loss_static": [_vp, _c_int, _vp, _vp, _vp, _vp, _vp, _vp, _c_int, _c_float, _c_int, _c_int, _c_int, _c_int,
                            _c_int, _c_float, _c_float, _c_int, _vp],
    "mi_tdt_forward": [_vp, _c_int, _vp, _vp, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _c_int, _c_float,
                       _c_float, _c_int, _c_int, _vp, _vp, _c_size_t, _vp],
    "mi_tdt_backward": [_vp, _c_int, _vp, _vp, _vp, _vp, _vp, _c_int, _c_float, _c_int, _c_int, _c_int, _c_int,
                        _c_int, _c_int, _vp, _c_int, _c_float, _c_float, _c_float, _c_int, _vp, _c_size_t, _vp],
    "mi_tdt_loss": [_vp, _c_int, _vp, _vp, _vp, _vp, _vp, _vp, _c_int, _c_float, _c_int, _c_int, _c_int, _c_int,
                    _c_int, _vp, _c_int, _c_float, _c_float, _c_float, _c_int, _c_int, _vp, _c_size_t, _vp],
    "mi_tdt_split_forward": [_vp, _vp, _c_int, _vp, _vp, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _c_int,
                             _c_float, _c_float, _c_int, _c_int, _vp, _vp, _c_size_t, _vp],
    "mi_tdt_split_backward": [_vp, _c_int, _vp, _vp, _vp, _vp, _vp, _vp, _c_int, _c_float, _c_int, _c_int, _c_int,
                              _c_int, _c_int, _c_int, _vp, _c_int, _c_float, _c_float, _c_float, _c_int, _vp,
                              _c_size_t, _vp],
    "mi_tdt_split_loss": [_vp, _vp, _c_int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _c_int, _c_float, _c_int, _c_int, _c_int,
                          _c_int, _c_int, _vp, _c_int, _c_float, _c_float, _c_float, _c_int, _c_int, _vp, _c_size_t, _vp],
    "mi_multiblank_forward": [_vp, _c_int, _vp, _vp, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _c_int,
                              _c_float, _c_float, _c_int, _vp, _vp, _c_size_t, _vp],
    "mi_multiblank_backward": [_vp, _c_int, _vp, _vp, _vp, _vp, _vp, _c_int, _c_float, _c_int, _c_int, _c_int, _c_int,
                               _c_int, _c_int, _vp, _c_int, _c_float, _c_float, _c_float, _vp, _c_size_t, _vp],
    "mi_multiblank_loss": [_vp, _c_int, _vp, _vp, _vp, _vp, _vp, _vp, _c_int, _c_float, _c_int, _c_int, _c_int, _c_int,
                           _c_int, _vp, _c_int, _c_float, _c_float, _c_float, _c_int, _vp, _c_size_t, _vp],
    "mi_rnnt_logprobs_forward": [_vp, _c_int, _vp, _vp, _vp, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _vp,
                                 _c_size_t, _vp],
    "mi_rnnt_logprobs_backward": [_vp, _c_int, _vp, _vp, _vp, _vp, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _c_int,
                                  _c_int, _vp, _c_size_t, _vp],
    "mi_joint_workspace_bytes": [_c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, ctypes.POINTER(_c_size_t)],
    "mi_joint_tile_bound": [_c_int, _c_int, _c_int],
    "mi_joint_rnnt_forward": [_vp, _vp, _vp, _vp, _c_int, _vp, _vp, _vp, _vp, _vp, _c_float, ctypes.c_uint64, _c_int,
                              _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _vp, _vp,
                              ctypes.c_longlong, _vp, _c_size_t, _vp],
    "mi_joint_tdt_forward": [_vp, _vp, _vp, _vp, _c_int, _vp, _vp, _vp, _vp, _vp, _c_float, ctypes.c_uint64, _c_int,
                             _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _c_int, _c_float, _c_float, _c_int, _vp,
                             _vp, ctypes.c_longlong, _vp, _c_size_t, _vp],
    "mi_joint_multiblank_forward": [_vp, _vp, _vp, _vp, _c_int, _vp, _vp, _vp, _vp, _vp, _c_float, ctypes.c_uint64,
                                    _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _c_int, _c_float, _c_float,
                                    _c_int, _vp, _vp, ctypes.c_longlong, _vp, _c_size_t, _vp],
    "mi_joint_dropout_mask": [_vp, _c_float, ctypes.c_uint64, _c_int, _c_int, _c_int, _c_int, _vp],
    "mi_joint_padded_vocabulary": [_c_int],
    "mi_joint_rnnt_backward": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _c_int, ctypes.c_longlong, _vp, _c_int, _c_float,
                               _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_float, _vp, _c_size_t, _vp],
    "mi_joint_tdt_backward": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _c_int, ctypes.c_longlong, _vp, _c_int, _c_float,
                              _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _c_int, _c_float, _c_float, _c_float,
                              _vp, _c_size_t, _vp],
    "mi_joint_multiblank_backward": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _c_int, ctypes.c_longlong, _vp, _c_int,
                                     _c_float, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _c_int, _c_float,
                                     _c_float, _c_float, _vp, _c_size_t, _vp],
    "mi_joint_reduce_hidden": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _c_int, _c_int, _c_float, ctypes.c_uint64, _c_int,
                               _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _vp, _c_size_t, _vp],
    "mi_joint_packed_weights": [_vp, _c_size_t, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                ctypes.POINTER(_vp),
                                ctypes.POINTER(_c_int), ctypes.POINTER(_c_int)],
    "mi_transducer_export_lattice": [_vp, _c_size_t, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _vp, _vp, _vp, _vp,
                                     _vp, _vp],
    "mi_transducer_length_maxima": [_vp, _vp, _c_int, _vp, _vp],
    "mi_transducer_denominators": [_vp, _c_int, _vp, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _vp,
                                   _c_size_t, _vp],
    "mi_rnnt_lattice": [_vp, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _c_float, _c_int, _vp, _c_size_t, _vp],
    "mi_tdt_lattice": [_vp, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _vp, _c_float, _c_float, _c_int, _vp, _c_size_t,
                       _vp],
    "mi_transducer_zero_padding": [_vp, _c_int, _vp, _vp, _c_int, _c_int, _c_int, _c_int, _vp],
    "mi_transducer_profile_enable": [_c_int, ctypes.c_uint],
    "mi_transducer_profile_read": [_c_int, ctypes.POINTER(_c_float), ctypes.POINTER(_c_int)],
    "mi_transducer_profile_disable": [],
    "mi_transducer_describe_plan": [_c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                    ctypes.c_char_p, _c_size_t],
    "mi_transducer_copy_probe": [_vp, _vp, _c_size_t, _vp],
    "mi_transducer_prefill_record": [_c_int, _c_int, _c_int, _c_int, _c_size_t, _vp, _vp, _vp],
}  # fmt: skip

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def lib():
    """The loaded library; raises if it is missing or of another ABI version."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP extension has not been built "
                "(run `python -c 'import __graft_entry__ as g; g.build()'`); there is no fallback path"
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = _c_int
        got = handle.mi_transducer_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"libmi_transducer.so has ABI version {got}, expected {ABI_VERSION}: rebuild it")
        _lib = handle
    return _lib


_cpu_lib = None

_fp, _i64p = _vp, _vp
_CPU_SIGNATURES = {
    "mi_transducer_cpu_abi_version": [],
    "mi_rnnt_cpu_workspace_bytes": [_c_int, _c_int, _c_int, ctypes.POINTER(_c_size_t)],
    "mi_rnnt_cpu_forward": [_fp, _i64p, _i64p, _i64p, _fp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _vp,
                            _c_size_t, _c_int],
    "mi_rnnt_cpu_backward": [_fp, _i64p, _i64p, _i64p, _fp, _fp, _c_int, _c_float, _c_int, _c_int, _c_int, _c_int,
                             _c_int, _c_float, _c_float, _c_int, _vp, _c_size_t, _c_int],
}  # fmt: skip
CPU_EXPORTED_SYMBOLS = tuple(_CPU_SIGNATURES)


def cpu_lib():
    """The loaded host library; raises if it is missing (there is no other CPU implementation to fall back to)."""
    global _cpu_lib
    if _cpu_lib is None:
        if not os.path.exists(CPU_LIB_PATH):
            raise RuntimeError(
                f"{CPU_LIB_PATH} is missing: the host library has not been built "
                "(run `python -c 'import __graft_entry__ as g; g.build()'`); there is no fallback path"
            )
        handle = ctypes.CDLL(CPU_LIB_PATH)
        for name, argtypes in _CPU_SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = _c_int
        got = handle.mi_transducer_cpu_abi_version()
        if got != CPU_ABI_VERSION:
            raise RuntimeError(f"libmi_transducer_cpu.so has ABI version {got}, expected {CPU_ABI_VERSION}: rebuild it")
        _cpu_lib = handle
    return _cpu_lib


def cpu_workspace_bytes(B, T, U):
    out = _c_size_t(0)
    if cpu_lib().mi_rnnt_cpu_workspace_bytes(B, T, U, ctypes.byref(out)) != SUCCESS:
        raise RuntimeError("Invalid parameter passed when calculating working space memory")  # rnnt.py:83-85
    return int(out.value)


def check_status(status, what):
    """Map the library's status codes to the reference's exception (rnnt.py:184-185, 219-234)."""
    if status == SUCCESS:
        return
    if status == INVALID_VALUE:
        raise RuntimeError(f"{what}: invalid value passed to the transducer-loss library")
    if status == TOO_LARGE:
        raise RuntimeError(
            f"{what}: the shape needs more than the {STATIC_WORKSPACE_BYTES >> 20} MiB workspace built into the "
            "library; use the entry point that takes a caller-owned workspace"
        )
    raise RuntimeError(f"{what}: HIP kernel launch failed (status {status})")


def workspace_bytes(B, T, U, D=0):
    out = _c_size_t(0)
    status = lib().mi_transducer_workspace_bytes(B, T, U, D, ctypes.byref(out))
    if status != SUCCESS:
        # rnnt.py:184-185
        raise RuntimeError("Invalid parameter passed when calculating working space memory")
    return int(out.value)


# pipeline stages that can be timed; which kernel runs a stage depends on the shape (describe_plan)
PROFILE_KERNELS = {
    "denominator_pass": 0,
    "lattice": 1,
    "cells": 2,
    "gradient_pass": 3,
    "zero_padding": 4,
    "weight_gradient": 5,
}


def describe_plan(dtype_code, B, T, U, V, D=0, max_duration=0, use_plain_rnnt=False, num_big_blanks=0):
    """{'denominators': kernel, 'lattice': kernel, 'cells': kernel or '-', 'gradient': kernel} for a shape
    (D > 0: TDT with that many durations; num_big_blanks > 0: multi-blank, V counting the big blanks)."""
    buf = ctypes.create_string_buffer(512)
    check_status(
        lib().mi_transducer_describe_plan(
            int(dtype_code), int(B), int(T), int(U), int(V), int(D), int(max_duration), int(bool(use_plain_rnnt)),
            int(num_big_blanks), buf, ctypes.c_size_t(len(buf)),
        ),
        "describe_plan",
    )
    return dict(item.split("=", 1) for item in buf.value.decode().split("; "))


def profile_enable(max_launches, kernels=None):
    """Bracket the next launches of the named kernels (default: all) with HIP events."""
    mask = 0
    for name in kernels or PROFILE_KERNELS:
        mask |= 1 << PROFILE_KERNELS[name]
    check_status(lib().mi_transducer_profile_enable(int(max_launches), mask), "profile_enable")


def profile_read():
    """{kernel: (total_ms, launches)} for the launches recorded since the last read."""
    out = {}
    for name, kid in PROFILE_KERNELS.items():
        ms, n = _c_float(0.0), _c_int(0)
        check_status(lib().mi_transducer_profile_read(kid, ctypes.byref(ms), ctypes.byref(n)), "profile_read")
        out[name] = (float(ms.value), int(n.value))
    return out


def profile_disable():
    check_status(lib().mi_transducer_profile_disable(), "profile_disable")
