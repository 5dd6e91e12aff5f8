"""The C-ABI library loads (no GPU needed for that) and exports every function include/*.h declares."""
import ctypes
import glob
import os
import re

from nnfusion_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    names = []
    for path in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = open(path).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"//[^\n]*", "", text)
        # a declaration: <type> nnf_name( ... );
        names += re.findall(r"\b(nnf_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_header_declares_the_expected_entry_points():
    names = _declared_functions()
    for must in ("nnf_w4a16_gemm", "nnf_w4a16_gemm_workspace_bytes", "nnf_w4a16_gemm_fused", "nnf_w8a8_gemm",
                 "nnf_w8a8_gemm_acc", "nnf_fused_mlp_w4a16", "nnf_status_string", "nnf_abi_version"):
        assert must in names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_lib.KERNELS_SO)
    missing = [n for n in _declared_functions() if not hasattr(lib, n)]
    assert not missing, missing


def test_library_exports_nothing_but_the_header():
    """Built with hidden visibility and a version script: the dynamic symbol table holds the header's functions only."""
    import subprocess

    out = subprocess.run(["nm", "-D", "--defined-only", _lib.KERNELS_SO], capture_output=True, text=True, check=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if line.split()[1:2] and line.split()[1] in "TW")
    assert exported == _declared_functions(), sorted(set(exported) ^ set(_declared_functions()))


def test_ctypes_table_covers_the_header():
    assert sorted(_lib.KERNEL_ABI) == _declared_functions()


def test_pure_host_queries_work_without_a_gpu():
    lib = _lib.kernels()
    assert lib.nnf_abi_version() == 4
    assert lib.nnf_status_string(0) == b"ok"
    assert b"workspace" in lib.nnf_status_string(-3)
    assert lib.nnf_w4a16_gemm_workspace_bytes(1, 4096, 4096, 128) == 0
    m, h, i = 256, 4096, 11008
    assert lib.nnf_fused_mlp_w4a16_workspace_bytes(m, h, i, 128) >= m * i * 2 + m * 4
    # decode-size fused calls: rstd (fp32 [M]) is the only scratch of the RMSNorm prologue, the gate | up pair needs none;
    # the MLP block adds its h tensor
    assert lib.nnf_w4a16_gemm_fused_workspace_bytes(1, 11008, 4096, 128, 1) == 256
    assert lib.nnf_w4a16_gemm_fused_workspace_bytes(16, 11008, 4096, 128, 1) == 256
    assert lib.nnf_w4a16_gemm_fused_workspace_bytes(1, 4096, 4096, 128, 0) == 256
    assert lib.nnf_fused_mlp_w4a16_workspace_bytes(1, 4096, 11008, 128) == 256 + 11008 * 2
    assert lib.nnf_fused_mlp_w4a16_workspace_bytes(256, 4096, 11008, 128) < 256 * 4096 * 2 + 256 * 11008 * 2 + (128 << 20)
    # variant / plan queries are host arithmetic too
    assert lib.nnf_w4a16_variant_supported(1, 4096, 4096, 128, 4) == 1 and lib.nnf_w4a16_variant_supported(64, 4096, 4096, 128, 4) == 0
    assert lib.nnf_w8a8_variant_supported(1, 4096, 4096, 3) == 1 and lib.nnf_w8a8_variant_supported(64, 4096, 4096, 1) == 0
    assert lib.nnf_w4a16_gemm_variant_workspace_bytes(4096, 8192, 8192, 128, 3, None) == 0
    # the general quantisation parameters: which combinations are served, and that only the specialised kernels use scratch
    from nnfusion_amd.ops import NnfQuant

    def qp(*f):
        q = NnfQuant(*f)
        return q, ctypes.cast(ctypes.pointer(q), ctypes.c_void_p)

    for fields, ok in (((4, 32, 8, None), 1), ((8, 128, 255, None), 1), ((8, 64, 256, None), 0), ((4, 16, 8, None), 0),
                       ((2, 32, 0, None), 0), ((4, 64, 16, None), 0)):
        keep, p = qp(*fields)
        assert lib.nnf_wna16_supported(8, 64, 256, p) == ok, fields
    keep, p = qp(4, 64, 8, None)
    assert lib.nnf_wna16_supported(8, 64, 96, p) == 0  # K % group
    # 4-bit weights above 16 rows: the tile GEMM's parked tiles; none for 8-bit weights, up to 16 rows, other K
    assert lib.nnf_wna16_gemm_workspace_bytes(128, 4096, 4096, p) == lib.nnf_w4a16_gemm_workspace_bytes(128, 4096, 4096, 128) > 0
    assert lib.nnf_wna16_gemm_workspace_bytes(16, 4096, 4096, p) == 0
    assert lib.nnf_wna16_gemm_workspace_bytes(128, 4096, 4096 + 64, p) == 0
    keep, p = qp(8, 64, 8, None)
    assert lib.nnf_wna16_gemm_workspace_bytes(128, 4096, 4096, p) == 0
    keep, p = qp(4, 128, 8, None)
    assert lib.nnf_wna16_gemm_workspace_bytes(128, 4096, 4096, p) == lib.nnf_w4a16_gemm_workspace_bytes(128, 4096, 4096, 128) > 0
    assert lib.nnf_wna16_gemm(None, None, None, None, None, 1, 64, 128, p, None, 0) == -1
    # argument checks come before any device access
    assert lib.nnf_w4a16_gemm(None, None, None, None, None, 1, 1, 128, 128, 8, None, 0) == -1
    assert lib.nnf_w8a8_gemm_acc(None, None, None, None, 1, 1, 128, None, 0) == -1


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    import pytest

    monkeypatch.setattr(_lib, "KERNELS_SO", str(tmp_path / "nope.so"))
    monkeypatch.setattr(_lib, "_kernels", None)
    with pytest.raises(_lib.NativeLibraryMissing):
        _lib.kernels()
