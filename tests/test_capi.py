"""The C-ABI library loads and exports every symbol include/iron_hip.h declares (no GPU needed)."""

import ctypes
import re
from pathlib import Path

from iron_amd import _lib

ROOT = Path(__file__).resolve().parent.parent


def declared_symbols():
    text = (ROOT / "include" / "iron_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(iron_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    handle = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared_symbols():
        assert hasattr(handle, name), name
    lib = _lib.lib()
    assert lib.iron_version() >= 100
    assert lib.iron_mha_decode_workspace_bytes(32, 64) == 32 * 128 * 66 * 4


def test_argument_refusals_need_no_gpu():
    """A refused call returns 1 before any launch and leaves its reason readable."""
    lib = _lib.lib()
    assert lib.iron_gemv_bf16(None, None, None, 8, 8, 1, 1, None, None) == 1
    assert b"null operand" in lib.iron_last_error()
    one = ctypes.c_void_p(16)
    assert lib.iron_gemv_bf16(one, one, one, 8, 12, 1, 1, None, None) == 1
    assert b"multiple of 8" in lib.iron_last_error()
    assert lib.iron_mha_prefill_bf16(one, one, one, one, 6, 4, 64, 8, 8, 8, 0.125, 1, -1, 0, 0, None, None, None) == 1
    assert b"multiple of kv_heads" in lib.iron_last_error()


def test_every_entry_point_refuses_null_operands():
    """Each entry point that takes pointers returns 1 with a reason, before any launch, when they
    are all null and every size is zero: nothing is dereferenced or launched on bad arguments."""
    lib = _lib.lib()
    for name, (_, args) in sorted(_lib.SIGNATURES.items()):
        if not any(a is _lib._P for a in args):
            continue
        call = [None if a is _lib._P else (0.0 if a is ctypes.c_float else 0) for a in args]
        assert getattr(lib, name)(*call) == 1, name
        assert lib.iron_last_error(), name


def test_bench_refuses_more_than_one_gpu():
    """``bench.py --gpus N`` with N above 1 exits with a message: this build is the one-GPU path."""
    import subprocess
    import sys
    from pathlib import Path

    bench = Path(__file__).resolve().parent.parent / "bench.py"
    done = subprocess.run([sys.executable, str(bench), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert done.returncode != 0 and "one-GPU" in done.stderr and done.stdout.strip() == ""
