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
    # pimdl_amm_desc: 8 x uint32 + float; pimdl_amm_timing: 3 floats
    assert ctypes.sizeof(pimdl.AmmDesc) == 36
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
