"""The C-ABI library loads on a machine without a GPU, exports every symbol the header declares,
and rejects bad arguments with AAMD_ERR_ARG before touching the device (no kernel is launched
by any call in this file)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "atorch_amd_fp8.h")
PROBES_HEADER = os.path.join(ROOT, "include", "atorch_amd_probes.h")


def _declared(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(aamd_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    from atorch_amd import _lib

    L = _lib.lib()
    names = _declared()
    assert len(names) >= 14
    for n in names:
        assert hasattr(L, n), f"{n} declared in the header but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names
    assert L.aamd_abi_version() == _lib.ABI_VERSION
    hdr = open(HEADER).read()
    assert f"#define AAMD_ABI_VERSION {_lib.ABI_VERSION}" in hdr


def test_every_entry_point_cites_the_reference():
    """Each declaration's comment names the reference file it replaces."""
    text = open(HEADER).read()
    for block in re.findall(r"/\*(.*?)\*/\s*(?:int64_t|int)\s+(aamd_[a-z0-9_]+)\s*\(", text, flags=re.S):
        comment, name = block
        if name == "aamd_abi_version":
            continue
        if "no counterpart in the reference" in comment:
            assert name == "aamd_grouped_gemm_fp8_nt_static", f"{name}: only the no-allocation entry may lack a counterpart"
            continue
        assert re.search(r"\.py:\d+", comment), f"{name}: no reference file:line in its comment"


def test_product_library_exports_only_the_header_and_no_measurement_aid():
    """Probes and launch-option pins live in libatorch_amd_probes.so; the product library exports exactly
    the entry points of its header."""
    import subprocess

    from atorch_amd import _lib, _probes

    out = subprocess.check_output(["nm", "-D", "--defined-only", _lib.LIB_PATH], text=True)
    exported = sorted(ln.split()[-1] for ln in out.splitlines() if ln.split()[-1].startswith("aamd_"))
    assert exported == _declared()
    assert not any("probe" in n or "tuning" in n or "option" in n for n in exported)
    P = _probes.lib()
    names = _declared(PROBES_HEADER)
    assert sorted(_probes.SIGNATURES) == names
    for n in names:
        assert hasattr(P, n), f"{n} declared in the probes header but not exported"
    assert not set(names) & set(_declared()), "the two libraries share no entry point"
    # the pinned GEMM validates like the product one, before touching the device
    one = ctypes.c_void_p(16)
    rc = P.aamd_tuning_grouped_gemm_fp8_nt(one, 64, one, one, one, 0, None, 1, None, 8, 128, 64, one, _lib.BF16, 128,
                                           None, _lib.NONE, _probes.options_array({"tile": 1}), None)
    assert rc == _lib.ERR_ARG and b"multiples of 128" in P.aamd_probes_last_error()


def test_argument_validation_without_gpu():
    from atorch_amd import _lib

    L = _lib.lib()
    one = ctypes.c_void_p(16)  # a non-null, 16-byte aligned fake address: validation fails before any use
    # cols not a multiple of 128
    rc = L.aamd_quant_1x128(one, _lib.BF16, 4, 100, 100, one, one, 0.0, None)
    assert rc == _lib.ERR_ARG and b"multiple of 128" in L.aamd_last_error()
    # unsupported dtype
    rc = L.aamd_quant_1x128(one, 7, 4, 128, 128, one, one, 0.0, None)
    assert rc == _lib.ERR_ARG and b"dtype" in L.aamd_last_error()
    # block quant needs both dims % 128
    rc = L.aamd_quant_128x128(one, _lib.BF16, 1, 100, 128, 12800, one, one, None, None, 0.0, None)
    assert rc == _lib.ERR_ARG
    # GEMM: K not a multiple of 128; grouped without offsets
    rc = L.aamd_grouped_gemm_fp8_nt(one, 64, one, one, one, 0, None, 1, None, 8, 128, 64, one, _lib.BF16, 128, None, _lib.NONE, None)
    assert rc == _lib.ERR_ARG
    rc = L.aamd_grouped_gemm_fp8_nt(one, 128, one, one, one, 0, None, 2, None, 8, 128, 128, one, _lib.BF16, 128, None, _lib.NONE, None)
    assert rc == _lib.ERR_ARG and b"group_offsets" in L.aamd_last_error()
    # unpermute: topk out of range, H not a multiple of 8
    rc = L.aamd_unpermute_combine(one, _lib.BF16, 8, 64, one, one, _lib.BF16, 4, 100, one, None)
    assert rc == _lib.ERR_ARG and b"topk" in L.aamd_last_error()
    rc = L.aamd_unpermute_combine(one, _lib.BF16, 8, 60, one, one, _lib.BF16, 4, 2, one, None)
    assert rc == _lib.ERR_ARG
    # preprocess: too many experts
    rc = L.aamd_moe_preprocess(one, 1, 8, 5000, one, one, one, one, None)
    assert rc == _lib.ERR_ARG
    # empty problems are fine and launch nothing
    assert L.aamd_quant_1x128(None, _lib.BF16, 0, 128, 128, None, None, 0.0, None) == _lib.OK
    assert L.aamd_grouped_gemm_fp8_nt(None, 128, None, None, None, 0, None, 1, None, 0, 128, 128, None, _lib.BF16, 128, None, _lib.NONE, None) == _lib.OK
    assert L.aamd_moe_preprocess_ws_ints(4096, 8) == 8 * 4 + 8


def test_python_wrappers_refuse_cpu_tensors():
    import torch

    from atorch_amd import kernels

    with pytest.raises(ValueError, match="GPU"):
        kernels.tile_quant(torch.zeros(4, 128, dtype=torch.bfloat16))
