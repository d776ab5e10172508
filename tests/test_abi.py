"""CPU-side checks of the C-ABI library: it loads, and exports every symbol the header declares.
No compute call is made here (there is no GPU in the CPU test run)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "deers_rocm.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(deers_rocm_\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for must in ("deers_rocm_init", "deers_rocm_available", "deers_rocm_sync",
                 "deers_rocm_last_error", "deers_rocm_alloc", "deers_rocm_free",
                 "deers_rocm_htod", "deers_rocm_dtoh", "deers_rocm_attn_fwd",
                 "deers_rocm_attn_bwd", "deers_rocm_attn_decode"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from deers_amd import rocm
    if not os.path.exists(rocm.LIB_PATH):
        pytest.fail(f"{rocm.LIB_PATH} not built; run `make -C deers_amd/csrc`")
    lib = ctypes.CDLL(rocm.LIB_PATH)
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_calls_before_init_fail_loudly_without_a_device():
    """Host logic: entry points refuse to run before init and say why."""
    from deers_amd import rocm
    lib = rocm.load()
    if rocm._inited:
        pytest.skip("runtime already initialised in this process")
    rc = lib.deers_rocm_sync()
    assert rc == 4  # DEERS_ROCM_ERR_NOT_INIT
    assert b"deers_rocm_init" in lib.deers_rocm_last_error()


def test_default_scale_matches_reference_rule():
    import numpy as np
    from deers_amd import rocm
    # 1/sqrt(D) in f64, narrowed to f32 (src/models/gpt.rs:139, src/storage.rs:115-117)
    assert rocm.default_scale(64) == 0.125
    assert rocm.default_scale(32) == float(np.float32(1.0 / np.sqrt(32.0)))
