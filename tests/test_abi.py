"""The C-ABI library builds, loads on a machine without a GPU, and exports every symbol the header declares."""
import ctypes
import re
from pathlib import Path

import pytest

from areal_amd import _native

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "areal_amd.h"


def declared_functions():
    text = HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(aa_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    names = declared_functions()
    for must in ("aa_logits_fwd", "aa_logits_bwd", "aa_logits_ppo_fused", "aa_rejection_sampling", "aa_ppo_loss",
                 "aa_masked_sum", "aa_lmhead_fwd", "aa_lmhead_bwd"):
        assert must in names


def test_library_exports_every_declared_symbol():
    assert _native.LIB_PATH.exists(), "build the library first: python -m areal_amd.build"
    lib = ctypes.CDLL(str(_native.LIB_PATH))
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in areal_amd.h but not exported"


def test_binding_covers_header_and_loads():
    assert sorted(_native.SIGNATURES) == declared_functions()
    lib = _native.load()
    assert lib.aa_version() >= 100
    assert lib.aa_status_string(0) == b"ok"
    assert lib.aa_status_string(1) == b"invalid argument"


def test_header_is_plain_c(tmp_path):
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "t.c"
    src.write_text(f'#include "{HEADER}"\nint main(void) {{ return AA_OK; }}\n')
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-fsyntax-only", str(src)], check=True)


def test_argument_validation_without_gpu():
    """Entry points reject bad arguments before touching the device."""
    lib = _native.load()
    null = ctypes.c_void_p(0)
    assert lib.aa_logits_fwd(null, 0, 1, 8, 8, null, 1.0, null, null, null, null, null, null, null) == 1
    assert lib.aa_copy_bytes(null, null, 16, null) == 1
    assert lib.aa_masked_sum(null, null, -1, null, null, null, null) == 1
