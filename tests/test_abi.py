"""The C-ABI library loads and exports every symbol that include/clt_hip.h declares
(no kernels are launched here; this runs without a GPU)."""
import ctypes
import os
import re

import crosslayer_coding_amd as cca
from crosslayer_coding_amd import _native as nat

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "clt_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(clt_[a-z_0-9]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(nat.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    lib = nat.load()
    raw = ctypes.CDLL(nat.library_path())
    for name in declared_symbols():
        assert hasattr(raw, name), name
    assert lib.clt_version() >= 100
    assert lib.clt_error_string(0) == b"ok"
    assert b"workspace" in lib.clt_error_string(-3)
    assert b"unknown" in lib.clt_error_string(-99)


def test_workspace_queries_and_argument_errors_need_no_gpu():
    lib = nat.load()
    n = lib.clt_batchtopk_workspace_bytes(4096, 24576, 12, 200, 0, 1)
    assert n > 12 * 4096 * 8 and n % 256 == 0
    assert lib.clt_batchtopk_workspace_bytes(4096, 24576, 12, 200, 1, 1) > 0
    # argument validation happens before any launch
    assert lib.clt_encode(None, None, None, None, 4, 8, 16, 1, 0, 0, 0, 0, 7, None) == -2
    assert lib.clt_encode(None, None, None, None, 4, 8, 16, 1, 0, 0, 0, 0, 0, None) == -1
    assert lib.clt_decode_sparse(None, None, None, None, None, None, None, None, None,
                                 4, 8, 16, 65, 0, 0, 1, 1, 0, 0, None, 0, None) == -1
    assert lib.clt_decode_workspace_bytes(4096, 768, 24576, 12) >= 8 * 12 * 4096 * 768 * 4
    assert lib.clt_pack_decoder(None, None, 8, 16, 1, 0, 0, 0, None) == -1


def test_no_cpu_fallback():
    import pytest
    import torch

    with pytest.raises(nat.CLTNativeError):
        cca.engine.encode(torch.zeros(1, 2, 8), torch.zeros(1, 4, 8), None)
    with pytest.raises(nat.CLTNativeError):
        cca.BatchTopK._compute_mask(torch.randn(2, 4), 2)


def test_encoder_kernels_spill_nothing(tmp_path):
    """Every instantiation of the matrix-core encoder kernel must fit the register file: the kernel runs two
    wavefronts per SIMD on 256 registers each, with 128 of them accumulators that live across the K loop, so a
    change that tips it into spilling costs the loop dearly while every result stays right.  Checked on the
    assembly the compiler reports for gfx950."""
    import shutil
    import subprocess

    import pytest
    from crosslayer_coding_amd import build as clt_build

    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not found")
    out = tmp_path / "encode.s"
    flags = [f for f in clt_build.HIP_FLAGS if f != "-fPIC"]
    proc = subprocess.run([hipcc, *flags, "--cuda-device-only", "-S", "-o", str(out),
                           os.path.join(clt_build.CSRC, "encode.hip")], stdout=subprocess.PIPE, stderr=subprocess.STDOUT,
                          text=True)
    assert proc.returncode == 0, proc.stdout[-2000:]
    current, scratch = None, {}
    for line in open(out):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            current = m.group(1)
        m = re.match(r"^; ScratchSize: (\d+)", line)
        if m and current:
            scratch[current] = int(m.group(1))
    kernels = {k: v for k, v in scratch.items() if "k_encode_mfma" in k}
    assert len(kernels) >= 18, sorted(kernels)      # 3 element types x 3 epilogues x even / odd stage counts, + segmented
    assert all(v == 0 for v in kernels.values()), {k: v for k, v in kernels.items() if v}
