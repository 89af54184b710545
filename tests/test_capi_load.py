"""CPU-side checks of the drop-in boundary: the C-ABI library loads and exports every symbol that
include/pimdl.h declares; with no GPU, initialisation fails loudly instead of falling back."""
import ctypes
import os
import re

import pytest

from __graft_entry__ import ROOT, load_package

pimdl = load_package()


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "pimdl.h")).read()
    return sorted(set(re.findall(r"PIMDL_API\s+[\w\s\*]+?\b(pimdl_\w+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared_symbols() == sorted(pimdl.EXPORTS)


def test_library_exports_every_declared_symbol():
    if not os.path.exists(pimdl.LIB_PATH):
        pytest.skip("libpimdl.so not built yet (run __graft_entry__.build())")
    lib = ctypes.CDLL(pimdl.LIB_PATH)
    for name in _declared_symbols():
        assert hasattr(lib, name), name


def test_struct_layouts_match_the_header():
    # pimdl_amm_desc: 8 x uint32 + float + uint32 (activation); pimdl_amm_timing: 3 floats
    assert ctypes.sizeof(pimdl.AmmDesc) == 40
    assert pimdl.AmmDesc.activation.offset == 36
    assert ctypes.sizeof(pimdl.AmmTiming) == 12
    assert ctypes.sizeof(pimdl.AmmGeometry) == 14 * 4
    assert ctypes.sizeof(pimdl.DeviceInfo) == 64 + 32 + 4 * 3 + 4 + 8  # 4 bytes of padding before the u64


def test_no_cpu_fallback_without_a_gpu():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    if not os.path.exists(pimdl.LIB_PATH):
        pytest.skip("libpimdl.so not built yet")
    with pytest.raises(pimdl.PimdlError) as e:
        pimdl.Context(0)
    assert e.value.code == -5 and "no CPU fallback" in str(e.value)


def test_host_layer_exports_the_reference_operator_api():
    """The C++ layer with the reference's names: amm_host, index_calculation, pim_lut and the DPU-set helpers."""
    import subprocess

    if not os.path.exists(pimdl.LIB_PATH):
        pytest.skip("libpimdl.so not built yet")
    out = subprocess.run(["nm", "-D", "--demangle", pimdl.LIB_PATH], capture_output=True, text=True).stdout
    for sig in ("amm_host(dpu_set_t*, float*, float*, signed char*, float*, float*, IndexCalcParams, LUTParams)",
                "index_calculation(float*, float*, unsigned short*, IndexCalcParams)",
                "pim_lut(LUTParams, dpu_set_t*, unsigned short*, signed char*, float*, float*)",
                "allocate_dpu(dpu_set_t*, unsigned int)", "allocate_rank(dpu_set_t*, unsigned int)",
                "free_dpu_set(dpu_set_t*)", "load_binary(dpu_set_t*, std::"):
        assert sig in out, sig


def test_reference_param_structs_keep_their_layout():
    """IndexCalcParams is 8 x uint32 and LUTParams 18 x 4 bytes, as in the reference's defines.h:12-50."""
    import subprocess
    import tempfile

    src = '#include "pimdl/defines.h"\n#include <cstdio>\n#include <cstddef>\nint main(){printf("%zu %zu %zu %zu %zu\\n", sizeof(IndexCalcParams), sizeof(LUTParams), offsetof(LUTParams, scale), offsetof(LUTParams, lut_load_type), sizeof(AMMParams));}\n'
    with tempfile.TemporaryDirectory() as d:
        open(os.path.join(d, "t.cpp"), "w").write(src)
        subprocess.check_call(["g++", "-std=c++11", "-I", os.path.join(ROOT, "include"), "-o", os.path.join(d, "t"),
                               os.path.join(d, "t.cpp")])
        out = subprocess.check_output([os.path.join(d, "t")], text=True).split()
    assert out == ["32", "72", "16", "60", "104"]
