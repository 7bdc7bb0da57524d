"""The C-ABI library loads without a GPU and exports every symbol include/ranncgrad.h declares."""
import ctypes
import os
import re

import pytest

from rannc_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ranncgrad.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b(rg_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in ("rg_fused_step", "rg_unscale_pack", "rg_grad_norm", "rg_scale_cast", "rg_zero",
                 "rg_plan_create", "rg_plan_destroy", "rg_segment_layout", "rg_bucket_layout",
                 "rg_aligned_numel", "rg_last_error"):
        assert must in names


@pytest.mark.parametrize("name", declared_functions())
def test_symbol_exported(name):
    lib = ctypes.CDLL(_lib.LIB_PATH)
    assert hasattr(lib, name), f"{name} declared in ranncgrad.h but not exported"


def test_binding_covers_header():
    assert sorted(_lib.SIGNATURES) == declared_functions()


def test_no_torch_types_in_header():
    text = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)   # declarations only
    assert "at::" not in text and "torch" not in text.lower() and "Tensor" not in text


def test_status_codes_become_python_exceptions():
    # bad arguments never reach the device
    assert _lib.lib.rg_aligned_numel(-1, 4, 1) == -1
    with pytest.raises(ValueError):
        _lib.aligned_numel(10, 3, 1)
    with pytest.raises(ValueError):
        _lib.segment_layout(10, 4, 0)
    with pytest.raises(ValueError):
        _lib.bucket_layout([1, 2], [0, 7])
    assert _lib.lib.rg_elem_size(_lib.RG_F32) == 4 and _lib.lib.rg_elem_size(_lib.RG_BF16) == 2
    assert _lib.lib.rg_elem_size(9) == -1
    assert _lib.lib.rg_plan_num_tensors(None) == -1


def test_plan_create_rejects_bad_arguments_before_touching_a_device():
    with pytest.raises(ValueError, match="chunk_elems"):
        _lib.Plan(0, [None], [None], [10], [0], [0], chunk_elems=1000)
    with pytest.raises(ValueError, match="dtype"):
        _lib.Plan(0, [None], [None], [10], [5], [0])
    with pytest.raises(ValueError, match="aligned"):
        _lib.Plan(0, [0x1001], [None], [10], [_lib.RG_F16], [_lib.RG_F16])
    with pytest.raises(ValueError, match="numel"):
        _lib.Plan(0, [None], [None], [-1], [0], [0])


def test_header_is_plain_c99():
    """The boundary is a C ABI: the header must compile as C99 (no C++ constructs, no torch or HIP types)."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    proc = subprocess.run([gcc, "-std=c99", "-pedantic", "-Wall", "-Werror", "-fsyntax-only", "-x", "c", HEADER],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout
