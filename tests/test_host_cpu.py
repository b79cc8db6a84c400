"""CPU-side checks of the shipped libraries: they load, export what the header declares,
and the host quantiser reproduces the numpy statement of the formula bit for bit.
No GPU call is made here."""
import ctypes as C
import importlib
import subprocess

import numpy as np

from synth import quantize_u8

fr = importlib.import_module("faster-rwkv_amd")


def test_libfrhip_exports_every_declared_symbol():
    lib = fr.lib()
    names = fr.declared_symbols()
    assert len(names) >= 40
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, "declared in include/frhip.h but not exported: %s" % missing
    assert lib.frhip_abi_version() == 1


def test_workspace_query_and_argument_checks_do_not_need_a_gpu():
    lib = fr.lib()
    assert lib.frhip_decode_workspace_bytes(2048, 8192) >= 2 * (3 * 2048 + 8192)
    assert lib.frhip_decode_workspace_bytes(0, 0) == 0
    assert lib.frhip_gemv(None, None, None, fr.F16, None) == -1  # FRHIP_EINVAL before any launch
    assert lib.frhip_layernorm(None, None, None, None, 1, 8, fr.F16, None) == -1
    assert b"null" in lib.frhip_error_string()


def test_host_library_loads_and_reports_errors_as_status():
    h = fr.host()
    m = h.fr_model_create(b"/nonexistent/model.fr", b"tpu fp16")
    assert not m
    assert b"unknown device" in h.fr_last_error()
    m = h.fr_model_create(b"/nonexistent/model.fr", b"cpu fp32")  # no CPU model path, as upstream
    assert not m and b"not found" in h.fr_last_error()


def test_host_quantiser_matches_numpy_statement_bit_for_bit():
    h = fr.host()
    rng = np.random.default_rng(5)
    for K, N in ((64, 48), (256, 320), (48, 1024)):
        w = (rng.standard_normal((K, N)) * 0.02).astype(np.float16)
        q = np.empty((K, N), np.uint8)
        mx, rx = np.empty(N, np.float16), np.empty(N, np.float16)
        my, ry = np.empty(K, np.float16), np.empty(K, np.float16)
        assert h.fr_quantize_u8(w.ctypes.data, K, N, q.ctypes.data, mx.ctypes.data, rx.ctypes.data,
                                my.ctypes.data, ry.ctypes.data) == 0
        rq, rmx, rrx, rmy, rry = quantize_u8(w)
        for a, b in ((mx, rmx), (rx, rrx), (my, rmy), (ry, rry)):
            assert np.array_equal(a.view(np.uint16), b.view(np.uint16))
        assert np.array_equal(q, rq)


def test_host_unit_tests_binary():
    """C++ unit tests of the host layer (float16 conversion, registry, reshape, msgpack,
    error macros); built by faster-rwkv_amd/host/Makefile."""
    import os
    exe = os.path.join(fr.HERE, "host_tests")
    assert os.path.exists(exe), "host_tests is not built"
    out = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "all host tests passed" in out.stdout
