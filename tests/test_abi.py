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


def test_count_on_device_marker_agrees_with_the_header(tmp_path):
    """``AA_LMHEAD_COUNT_ON_DEVICE`` of the binding is the header's: a C program prints the macro."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src, exe = tmp_path / "m.c", tmp_path / "m"
    src.write_text(f'#include <stdio.h>\n#include "{HEADER}"\n'
                   'int main(void) { printf("%lld\\n", (long long)AA_LMHEAD_COUNT_ON_DEVICE); return 0; }\n')
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    assert int(out) == _native.AA_LMHEAD_COUNT_ON_DEVICE


def test_argument_validation_without_gpu():
    """Entry points reject bad arguments before touching the device."""
    lib = _native.load()
    null = ctypes.c_void_p(0)
    assert lib.aa_logits_fwd(null, 0, 1, 8, 8, null, 1.0, null, null, null, null, null, null, null) == 1
    assert lib.aa_copy_bytes(null, null, 16, null) == 1
    assert lib.aa_masked_sum(null, null, -1, null, null, null, null) == 1


def test_argument_validation_of_the_sibling_entry_points_without_gpu():
    """The losses, reductions and layout entry points return AA_ERR_INVALID_ARGUMENT (or AA_OK for empty input) before
    any launch: null outputs, negative sizes, enum values out of range."""
    lib = _native.load()
    z = ctypes.c_void_p(0)
    p = ctypes.c_void_p(256)        # a non-null address that is never dereferenced on the host
    bad, ok = 1, 0
    assert lib.aa_kl_estimate(p, p, -1, 0, 0, p, z) == bad
    assert lib.aa_kl_estimate(p, p, 4, 3, 0, p, z) == bad
    assert lib.aa_kl_estimate(z, z, 0, 0, 0, z, z) == ok
    assert lib.aa_dpo_seq_sums(p, p, p, p, -1, 4, p, p, p, z) == bad
    assert lib.aa_dpo_seq_sums(p, p, p, z, 2, 4, p, p, p, z) == bad
    assert lib.aa_dpo_seq_sums(z, z, z, z, 0, 0, z, z, z, z) == ok
    assert lib.aa_dpo_seq_sums_bwd(z, z, p, p, 2, 4, p, z) == bad
    assert lib.aa_dpo_preference_loss(p, 4, 0.1, 2, p, z, z) == bad
    assert lib.aa_dpo_preference_loss(p, 4, 0.1, 0, z, z, z) == bad
    assert lib.aa_dpo_preference_loss(z, 0, 0.1, 0, z, z, z) == ok
    assert lib.aa_dpo_pair_loss(p, p, p, p, 2, 0.1, 0, z, p, p, p, p, p, p, z) == bad
    assert lib.aa_dpo_pair_loss(p, p, p, p, 2, 0.1, 5, p, p, p, p, p, p, p, z) == bad
    assert lib.aa_rw_pair_loss(p, 4, z, 1, p, p, p, p, p, p, z, z) == bad
    assert lib.aa_rw_pair_loss(z, 4, p, 1, p, p, p, p, p, p, z, z) == bad
    assert lib.aa_sft_loss(p, p, 4, z, 2, p, z, p, z, z, p, p, z, z) == bad       # sequences without cu_seqlens
    assert lib.aa_sft_loss(p, p, 4, p, 2, z, z, p, z, z, p, p, z, z) == bad       # no token count
    assert lib.aa_sft_loss(z, z, 4, p, 2, p, z, p, z, z, p, p, z, z) == bad
    assert lib.aa_logging_stats(p, p, z, z, p, 4, 0, 1, 0, p, p, 1 << 20, z) == bad    # a method without versions
    assert lib.aa_logging_stats(p, p, z, p, p, 4, 0, 7, 1, p, p, 1 << 20, z) == bad    # errors without ground truth
    assert lib.aa_logging_stats(p, p, z, p, p, 4, 0, 8, 0, p, p, 1 << 20, z) == bad
    assert lib.aa_logging_stats(p, p, z, p, p, 4, 0, 1, 0, p, p, 8, z) == bad          # scratch too small
    assert lib.aa_logging_stats_scratch_bytes(-1) == -1 and lib.aa_logging_stats_scratch_bytes(100000) > 0
    assert lib.aa_masked_normalization(p, z, 2, 8, 0, 1e-5, p, p, 8, z) == bad         # scratch too small
    assert lib.aa_masked_normalization(z, z, 0, 8, 0, 1e-5, z, z, 0, z) == ok
    assert lib.aa_masked_normalization_scratch_bytes(4, -1) == -1
    assert lib.aa_overlong_penalty(p, p, 4, 8, 0, 1.0, 100, z) == bad                   # division by overlong_tokens
    assert lib.aa_kd_terms(p, z, p, p, 4, 1, p, p, z) == bad                            # pure form without old log-probs
    assert lib.aa_vocab_partials_combine(p, p, p, 0, 4, p, z, z, z, z) == bad       # no slice
    assert lib.aa_vocab_partials_combine(z, p, p, 2, 4, p, z, z, z, z) == bad
    assert lib.aa_vocab_partials_combine(z, z, z, 2, 0, p, z, z, z, z) == ok
    params = _native.PpoParams(clip_lo=0.8, clip_hi=1.2, loss_kind=7)
    assert lib.aa_logits_ppo_fused(p, 0, 4, 4096, 4096, p, 1.0, 4, p, p, p, z, ctypes.byref(params), p, z, p, z, z, z,
                                   p, p, p, p, z, z) == bad                             # unknown loss kind
    params = _native.PpoParams(loss_kind=2, sapo_tau_pos=1.0, sapo_tau_neg=0.0)
    assert lib.aa_logits_ppo_fused(p, 0, 4, 4096, 4096, p, 1.0, 4, p, p, p, z, ctypes.byref(params), p, z, p, z, z, z,
                                   p, p, p, p, z, z) == bad                             # SAPO gate temperature of zero
    params = _native.PpoParams(clip_lo=0.8, clip_hi=1.2, loss_kind=1)
    assert lib.aa_ppo_loss(p, p, p, p, z, 4, z, 0, 0, ctypes.byref(params), p, p, p, p, p, z) == 2   # unsupported
