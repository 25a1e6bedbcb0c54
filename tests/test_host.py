"""CPU-side checks: the C-ABI library loads and exports every declared symbol,
the host-side validation mirrors the reference, and nothing in the package
reaches for the oracle."""

import os
import re

import numpy as np
import pytest
import torch

from speech_amd import _native
from speech_amd.rnnt_loss.rnnt_pytorch import RNNTLossNumba, TDTLossNumba, certify_inputs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def built_lib():
    if not os.path.exists(_native.LIB_PATH):
        _native.build()
    return _native.lib()


def test_library_exports_every_symbol_declared_in_the_header(built_lib):
    header = open(os.path.join(ROOT, "include", "mi_transducer.h")).read()
    declared = set(re.findall(r"^int (mi_[a-z_]+)\(", header, flags=re.M))
    assert declared == set(_native.EXPORTED_SYMBOLS)
    for name in declared:
        assert hasattr(built_lib, name), name
    assert built_lib.mi_transducer_abi_version() == _native.ABI_VERSION


def test_workspace_size_and_invalid_dimensions(built_lib):
    small = _native.workspace_bytes(1, 2, 3, 0)
    big = _native.workspace_bytes(16, 375, 121, 0)
    assert 0 < small < big
    assert _native.workspace_bytes(16, 375, 121, 5) > big
    # utils/rnnt_helper.py:119-142: any non-positive dimension is an invalid value -> RuntimeError (rnnt.py:184-185)
    for dims in [(0, 2, 3, 0), (1, 0, 3, 0), (1, 2, 0, 0), (1, 2, 1025, 0), (1, 2, 3, 17)]:
        with pytest.raises(RuntimeError):
            _native.workspace_bytes(*dims)


def test_null_and_bad_arguments_return_invalid_value_without_touching_the_gpu(built_lib):
    # every check happens on the host before any HIP call
    assert built_lib.mi_rnnt_forward(None, 0, None, None, None, None, 1, 2, 3, 4, 0, 0.0, 0, None, None, 0, None) == 1
    assert built_lib.mi_tdt_forward(None, 0, None, None, None, None, 1, 2, 3, 4, 2, None, 0, 0.0, 0.0, 0, 0, None, None, 0, None) == 1
    assert built_lib.mi_transducer_length_maxima(None, None, 1, None, None) == 1


def test_kernel_plan_of_the_documented_shapes(built_lib):
    """Which kernel family a shape maps to (host logic only: nothing is launched)."""
    F32, BF16 = 0, 1
    plan = _native.describe_plan
    p = plan(F32, 16, 375, 121, 1025)  # the benchmark shape: 256 whole vectors per row
    assert p == {
        "denominators": "denom_rows_kernel<f32, R=4, RPW=1>",
        "lattice": "rnnt_lattice_kernel<K=2>",
        "cells": "-",
        "gradient": "grad_block_kernel<f32, RT=128, NVT=2, fused>",
    }
    p = plan(BF16, 32, 750, 201, 1025)  # 128 whole vectors of 8 bf16
    assert p["denominators"] == "denom_rows_kernel<bf16, R=2, RPW=2>" and p["lattice"] == "rnnt_lattice_kernel<K=4>"
    assert p["gradient"] == "grad_block_kernel<bf16, RT=64, NVT=2, fused>"
    p = plan(F32, 8, 250, 101, 16385)  # 4096 vectors: a workgroup per row
    assert p["denominators"] == "denom_block_kernel<f32, RT=1024, NVT=4>"
    assert p["gradient"] == "grad_block_kernel<f32, RT=1024, NVT=4, fused>"
    p = plan(F32, 4, 50, 21, 29)  # character vocabulary: short rows, coefficients from the cell kernel
    assert p["denominators"] == "denom_rows_kernel<f32, R=1, RPW=4>" and p["gradient"] == "grad_rows_kernel<f32, R=1, coef>"
    assert p["cells"] == "rnnt_cell_kernel"
    p = plan(F32, 2, 10, 5, 40001)  # beyond 8 vectors per thread: the streaming kernels with a running max
    assert p["denominators"] == "denom_gather_kernel<f32>" and p["gradient"] == "grad_stream_kernel<f32>"
    assert p["cells"] == "rnnt_cell_kernel"
    p = plan(F32, 16, 375, 121, 1025, D=5, max_duration=4)  # TDT: coefficients come from the cell kernel
    assert p["lattice"] == "tdt_lattice_pair_kernel<D=5>" and p["cells"] == "tdt_cell_kernel"
    assert p["gradient"] == "grad_block_kernel<f32, RT=128, NVT=2, coef>"
    p = plan(F32, 16, 375, 121, 1025, D=5, max_duration=4, use_plain_rnnt=True)
    assert p["lattice"] == "rnnt_lattice_kernel<K=2>" and p["cells"] == "-"
    p = plan(F32, 16, 375, 121, 1028, num_big_blanks=3)  # multi-blank: three big blanks inside V
    assert p["lattice"] == "multiblank_lattice_kernel<NBC=4>" and p["cells"] == "multiblank_cell_kernel"
    # 257 whole vectors, one past a power of two: 5 vectors per lane in pass 1, a third (nearly empty) vector per
    # thread in the gradient pass rather than twice the threads
    assert p["denominators"] == "denom_rows_kernel<f32, R=5, RPW=1>"
    # (that kernel writes the big blanks' entries itself; only the other gradient kernels are followed by a fix-up)
    assert p["gradient"] == "grad_block_kernel<f32, RT=128, NVT=3, coef>"
    p = plan(F32, 4, 50, 21, 32, num_big_blanks=3)  # short rows: the wave-per-row kernel, then the fix-up kernel
    assert p["gradient"] == "grad_rows_kernel<f32, R=1, coef> + multiblank_fixup_kernel"
    p = plan(F32, 2, 50, 1024, 1028, max_duration=8, num_big_blanks=3)  # ring of 9 x 6 x 1024 doubles > 160 KB of LDS
    assert p["lattice"] == "multiblank_lattice_pull_kernel"
    p = plan(F32, 2, 50, 513, 1025, D=9, max_duration=8)  # beyond 256 label columns: a wave per direction
    assert p["lattice"].startswith("tdt_lattice_kernel<K=")
    with pytest.raises(RuntimeError):
        plan(7, 1, 1, 1, 5)
    with pytest.raises(RuntimeError):
        plan(F32, 1, 4, 2, 9, D=2, max_duration=1, num_big_blanks=2)  # TDT and multi-blank exclude each other


def test_constructor_attributes_match_the_reference_conventions():
    loss = RNNTLossNumba()
    assert (loss.blank, loss.reduction, loss.fastemit_lambda, loss.clamp) == (0, 'mean', 0.0, 0.0)
    assert RNNTLossNumba(clamp=2).clamp == 2.0 and RNNTLossNumba(clamp=-1).clamp == 0.0
    tdt = TDTLossNumba(blank=5)
    assert tdt.durations == [] and tdt.sigma == 0.0 and tdt.omega == 0.0
    loss.reduction = None  # the outer wrapper mutates these (nemo/collections/asr/losses/rnnt.py:484-491)
    loss.blank = 3


def test_certify_inputs_on_cpu_tensors():
    acts = torch.zeros(2, 4, 3, 5)
    labels = torch.ones(2, 2, dtype=torch.int64)
    act_lens = torch.tensor([4, 3])
    label_lens = torch.tensor([2, 1])
    certify_inputs(acts, labels, act_lens, label_lens)
    with pytest.raises(TypeError, match="labels must be"):
        certify_inputs(acts, labels.int(), act_lens, label_lens)
    with pytest.raises(TypeError, match="label_lengths must be"):
        certify_inputs(acts, labels, act_lens, label_lens.int())
    with pytest.raises(ValueError, match="log_probs must be contiguous"):
        certify_inputs(acts.transpose(0, 1), labels, act_lens, label_lens)
    with pytest.raises(ValueError, match="log_probs must be 4D"):
        certify_inputs(acts[0], labels, act_lens[:1].repeat(4), label_lens[:1].repeat(4))
    with pytest.raises(ValueError, match="Input length mismatch"):
        certify_inputs(acts, labels, act_lens - 1, label_lens)
    with pytest.raises(ValueError, match="Output length mismatch"):
        certify_inputs(acts, labels, act_lens, label_lens - 1)


def test_cpu_tensors_take_the_host_library_and_tdt_refuses_them():
    acts = torch.zeros(1, 2, 2, 3, requires_grad=True)
    labels = torch.ones(1, 1, dtype=torch.int64)
    # all-zero logits, V = 3: every path has probability 3^-(T + U - 1) and there are 2 of them
    costs = RNNTLossNumba(reduction='none')(acts, labels, torch.tensor([2]), torch.tensor([1]))
    np.testing.assert_allclose(costs.detach().numpy(), [3 * np.log(3.0) - np.log(2.0)], rtol=1e-6)
    with pytest.raises(ValueError, match="non CUDA"):  # rnnt_pytorch.py:137-140
        TDTLossNumba(blank=0, durations=[0, 1])(acts, labels, torch.tensor([2]), torch.tensor([1]))


def test_host_library_exports_every_symbol_declared_in_its_header():
    header = open(os.path.join(ROOT, "include", "mi_transducer_cpu.h")).read()
    declared = set(re.findall(r"^int (mi_[a-z_]+)\(", header, flags=re.M))
    assert declared == set(_native.CPU_EXPORTED_SYMBOLS)
    if not os.path.exists(_native.CPU_LIB_PATH):
        _native.build_cpu()
    handle = _native.cpu_lib()
    for name in declared:
        assert hasattr(handle, name), name
    assert handle.mi_transducer_cpu_abi_version() == _native.CPU_ABI_VERSION
    with pytest.raises(RuntimeError):
        _native.cpu_workspace_bytes(0, 2, 3)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_native, "LIB_PATH", str(tmp_path / "libmi_transducer.so"))
    monkeypatch.setattr(_native, "_lib", None)
    with pytest.raises(RuntimeError, match="no fallback"):
        _native.lib()


def test_package_never_imports_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "speech_amd")):
        for name in files:
            if name.endswith((".py", ".hip", ".h", ".inc", ".cpp")):
                text = open(os.path.join(dirpath, name)).read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, name)
