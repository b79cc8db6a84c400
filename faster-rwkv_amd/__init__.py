"""Python-side loader of the MI355X RWKV backend.

Two shared libraries live in this directory:
  libfrhip.so     -- the gfx950 kernels behind the C ABI of include/frhip.h
  libfr_host.so   -- the C++ host layer (Tensor / registry / Model with the `hip`
                     device registered) and its small C API for scripts

This module only binds them with ctypes; all computation happens in the libraries.
Nothing here falls back to another implementation: if a library is missing the
import of the corresponding binding raises.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIBFRHIP = os.path.join(HERE, "libfrhip.so")
LIBHOST = os.path.join(HERE, "libfr_host.so")

F32, F16, U8 = 0, 1, 2
H2D, D2H, D2D = 0, 1, 2


class FrhipError(RuntimeError):
    pass


def build(verbose=False):
    """Compile both libraries in-tree (hipcc cross-compiles gfx950 without a GPU)."""
    out = None if verbose else subprocess.DEVNULL
    subprocess.check_call(["make", "-s", "-j8", "-C", os.path.join(HERE, "csrc")], stdout=out)
    host_dir = os.path.join(HERE, "host")
    if os.path.exists(os.path.join(host_dir, "Makefile")):
        subprocess.check_call(["make", "-s", "-j8", "-C", host_dir], stdout=out)


class Weight(C.Structure):
    """struct frhip_weight"""
    _fields_ = [("data", C.c_void_p), ("mx", C.c_void_p), ("rx", C.c_void_p), ("my", C.c_void_p),
                ("ry", C.c_void_p), ("K", C.c_int32), ("N", C.c_int32), ("dtype", C.c_int32)]


_vp, _i, _sz = C.c_void_p, C.c_int, C.c_size_t
_WP = C.POINTER(Weight)

_SIGS = {
    "frhip_abi_version": (_i, []),
    "frhip_error_string": (C.c_char_p, []),
    "frhip_device_count": (_i, [C.POINTER(_i)]),
    "frhip_init": (_i, [_i]),
    "frhip_device_info": (_i, [C.c_char_p, _sz, C.POINTER(_i), C.POINTER(_sz)]),
    "frhip_malloc": (_i, [C.POINTER(_vp), _sz]),
    "frhip_free": (_i, [_vp]),
    "frhip_host_malloc": (_i, [C.POINTER(_vp), _sz]),
    "frhip_host_free": (_i, [_vp]),
    "frhip_memcpy": (_i, [_vp, _vp, _sz, _i]),
    "frhip_memcpy_async": (_i, [_vp, _vp, _sz, _i, _vp]),
    "frhip_memset_async": (_i, [_vp, _i, _sz, _vp]),
    "frhip_stream_create": (_i, [C.POINTER(_vp)]),
    "frhip_stream_destroy": (_i, [_vp]),
    "frhip_stream_sync": (_i, [_vp]),
    "frhip_device_sync": (_i, []),
    "frhip_event_create": (_i, [C.POINTER(_vp)]),
    "frhip_event_destroy": (_i, [_vp]),
    "frhip_event_record": (_i, [_vp, _vp]),
    "frhip_event_sync": (_i, [_vp]),
    "frhip_event_elapsed_ms": (_i, [_vp, _vp, C.POINTER(C.c_float)]),
    "frhip_graph_begin": (_i, [_vp]),
    "frhip_graph_end": (_i, [_vp, C.POINTER(_vp)]),
    "frhip_graph_launch": (_i, [_vp, _vp]),
    "frhip_graph_destroy": (_i, [_vp]),
    "frhip_pack_transpose": (_i, [_vp, _vp, _i, _i, _i, _vp]),
    "frhip_dequant_u8": (_i, [_WP, _vp, _vp]),
    "frhip_layernorm": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "frhip_groupnorm_f32": (_i, [_vp, _i, _vp, _vp, _vp, _i, _i, _vp]),
    "frhip_gemv": (_i, [_vp, _WP, _vp, _i, _vp]),
    "frhip_cast": (_i, [_vp, _i, _vp, _i, _sz, _vp]),
    "frhip_fill": (_i, [_vp, _i, C.c_float, _sz, _vp]),
    "frhip_scalar_div_f16": (_i, [_vp, C.c_float, _sz, _vp]),
    "frhip_gather_rows": (_i, [_vp, _vp, _vp, _i, _i, _vp]),
    "frhip_decode_workspace_bytes": (_sz, [_i, _i]),
    "frhip_att_one_v4": (_i, [_i] + [_vp] * 12 + [_WP] * 4 + [_vp] * 7),
    "frhip_ffn_one": (_i, [_i, _i] + [_vp] * 6 + [_WP] * 3 + [_vp, _vp, _i, _vp, _vp]),
    "frhip_head": (_i, [_i, _vp, _vp, _vp, _WP, _vp, _vp]),
    "frhip_argmax_f32": (_i, [_vp, _i, _vp, _vp]),
}

_lib = None


def declared_symbols():
    """Entry points the header include/frhip.h declares (parsed from the header)."""
    import re
    text = open(os.path.join(ROOT, "include", "frhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(frhip_[a-z0-9_]+)\s*\(", text)))


def lib():
    """The loaded libfrhip.so (raises if it has not been built)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIBFRHIP):
            raise FrhipError("libfrhip.so is not built: run `python -c 'import __graft_entry__ as g; g.build()'`")
        _lib = C.CDLL(LIBFRHIP)
        for name, (res, args) in _SIGS.items():
            if hasattr(_lib, name):
                f = getattr(_lib, name)
                f.restype, f.argtypes = res, args
    return _lib


def check(code, what=""):
    if code != 0:
        raise FrhipError("%s failed (%d): %s" % (what or "frhip call", code, lib().frhip_error_string().decode()))


_inited = False


def init(device=0):
    global _inited
    if not _inited:
        check(lib().frhip_init(device), "frhip_init")
        _inited = True


class DevBuf:
    """A device allocation made through the C ABI, with numpy upload/download."""

    def __init__(self, nbytes):
        init()
        self.nbytes = int(nbytes)
        p = _vp()
        check(lib().frhip_malloc(C.byref(p), max(self.nbytes, 16)), "frhip_malloc")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        b.dtype, b.shape = a.dtype, a.shape
        if a.nbytes:
            check(lib().frhip_memcpy(b.ptr, a.ctypes.data, a.nbytes, H2D), "H2D")
        return b

    @classmethod
    def empty(cls, shape, dtype):
        dtype = np.dtype(dtype)
        shape = tuple(np.atleast_1d(shape).tolist())
        b = cls(int(np.prod(shape)) * dtype.itemsize)
        b.dtype, b.shape = dtype, shape
        return b

    def numpy(self):
        out = np.empty(self.shape, self.dtype)
        if out.nbytes:
            check(lib().frhip_memcpy(out.ctypes.data, self.ptr, out.nbytes, D2H), "D2H")
        return out

    def upload(self, a):
        a = np.ascontiguousarray(a, self.dtype)
        assert a.nbytes == self.nbytes
        check(lib().frhip_memcpy(self.ptr, a.ctypes.data, a.nbytes, H2D), "H2D")

    def free(self):
        if getattr(self, "ptr", None):
            lib().frhip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class PackedWeight:
    """A matrix weight on the device in the kernels' output-major layout, built from
    the reference's [K, N] array (binary16) or from uint8 codes plus mx/rx/my/ry."""

    def __init__(self, w_kn=None, q=None, mx=None, rx=None, my=None, ry=None):
        init()
        if w_kn is not None:
            w_kn = np.ascontiguousarray(w_kn, np.float16)
            K, N = w_kn.shape
            src = DevBuf.from_numpy(w_kn)
            self.data = DevBuf.empty((N, K), np.float16)
            check(lib().frhip_pack_transpose(src.ptr, self.data.ptr, K, N, 2, None), "pack")
            self.scales = []
            self.c = Weight(self.data.ptr, None, None, None, None, K, N, F16)
        else:
            q = np.ascontiguousarray(q, np.uint8)
            K, N = q.shape
            src = DevBuf.from_numpy(q)
            self.data = DevBuf.empty((N, K), np.uint8)
            check(lib().frhip_pack_transpose(src.ptr, self.data.ptr, K, N, 1, None), "pack")
            self.scales = [DevBuf.from_numpy(np.ascontiguousarray(v, np.float16)) for v in (mx, rx, my, ry)]
            self.c = Weight(self.data.ptr, self.scales[0].ptr, self.scales[1].ptr, self.scales[2].ptr,
                            self.scales[3].ptr, K, N, U8)
        check(lib().frhip_device_sync(), "sync")
        src.free()
        self.K, self.N = K, N

    @property
    def ref(self):
        return C.byref(self.c)
