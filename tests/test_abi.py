"""The C-ABI library loads and exports every function include/*.h declares (no GPU needed)."""
import numpy as np
import ctypes
import glob
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    names = []
    for h in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        names += re.findall(r"^\s*ORNITH_API\s+(?:const\s+)?(?:int|char\s*\*|void)\s*\*?\s*(ornith_\w+)\s*\(", text, flags=re.M)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    lib_path = os.path.join(ROOT, "ornith-rs_amd", "libornith_hip.so")
    assert os.path.exists(lib_path), "build it first: python ornith-rs_amd/build.py"
    lib = ctypes.CDLL(lib_path)
    names = declared_functions()
    assert len(names) >= 15
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_binding_fails_loudly_without_library(orn, monkeypatch):
    monkeypatch.setattr(orn, "_lib", None)
    monkeypatch.setattr(orn, "LIB_PATH", "/nonexistent/libornith_hip.so")
    try:
        orn.lib()
    except orn.OrnithError as e:
        assert "no CPU fallback" in str(e)
    else:
        raise AssertionError("missing library did not raise")


def test_error_path_reports_message_without_gpu(orn):
    # argument validation happens before any HIP call
    rc = orn.lib().ornith_kmatrix_check(None, 0, 0, 0)
    assert rc == 1
    assert b"null matrix" in orn.lib().ornith_last_error()
    s = orn.KMatrixStruct(orn.Q4K, 1, 4, 300, 1, 1, 1)
    assert orn.lib().ornith_kmatrix_check(ctypes.byref(s), 0, 0, 0) == 1
    assert b"multiple of 256" in orn.lib().ornith_last_error()
    s = orn.KMatrixStruct(orn.Q4K, 1, 4, 512, 1, 1, 1)
    assert orn.lib().ornith_kmatrix_check(ctypes.byref(s), ctypes.c_size_t(4 * 2 * 128), ctypes.c_size_t(4 * 2 * 12), ctypes.c_size_t(4 * 2 * 4)) == 0
    assert orn.lib().ornith_kmatrix_check(ctypes.byref(s), ctypes.c_size_t(4 * 2 * 128), ctypes.c_size_t(4 * 2 * 16), ctypes.c_size_t(4 * 2 * 4)) == 1


def test_host_random_functions_match_known_answers():
    """The key sequence is host code inside the library: threefry2x32-20 against the
    published Random123 vectors (through bits(), whose first word of a 2-word request is
    x of hash(key, (0, 1))), and the split against the oracle."""
    import importlib
    import util
    orn = importlib.import_module("ornith-rs_amd")
    assert orn.random_key(0x0123456789ABCDEF) == [0x01234567, 0x89ABCDEF]
    for key in ([0, 0], [0xFFFFFFFF, 0xFFFFFFFF], [0x13198A2E, 0x03707344]):
        for n in (1, 2, 3, 4, 9):
            assert np.array_equal(orn.random_bits(key, n), util.orc_random_bits(key, n))
        st, sub = orn.random_split(key)
        assert (st, sub) == tuple(util.orc_key_next(key))
    # a direct known answer: counter (0, 1) under key (0, 0) is not in the KAT list, but n = 2 with
    # key = KAT key and the oracle (itself pinned on the three KATs) covers the layout; and here
    # the one KAT that bits() can reach directly: n = 1 hashes (0, 0)
    assert orn.random_bits([0, 0], 1)[0] == 0x6B200159


def test_host_philox_matches_known_answers(orn):
    """Philox4x32-10 is host code inside the library: the published Random123 vectors."""
    assert orn.philox4x32_10([0, 0, 0, 0], [0, 0]) == [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert orn.philox4x32_10([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2) == [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]
    assert orn.philox4x32_10([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0]) == \
        [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]


def test_bench_refuses_more_than_one_gpu():
    """One GPU only: `bench.py --gpus N` with N > 1 exits with a message that says so, before
    anything touches a device."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stderr + r.stdout)
