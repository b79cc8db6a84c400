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
# FRHIP_LIBRARY: another build of the same library (the measurement build libfrhip_timeline.so, see timeline.py)
LIBFRHIP = os.environ.get("FRHIP_LIBRARY") or os.path.join(HERE, "libfrhip.so")
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
    "frhip_slice": (_i, [_vp, _vp, _i, _vp, _vp, _vp, _vp, _i, _vp]),
    "frhip_cat": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _sz, _i, _vp]),
    "frhip_transpose": (_i, [_vp, _vp, _i, _vp, _i, _i, _i, _vp]),
    "frhip_silu": (_i, [_vp, _vp, _i, _sz, _vp]),
    "frhip_embed_ring": (_i, [_vp, _i, _i, _vp, _i, _vp, _vp, _vp]),
    "frhip_embed_argmax": (_i, [_vp, _i, _i, _vp, _i, _vp, _i, _vp, _vp, _vp]),
    "frhip_decode_workspace_bytes": (_sz, [_i, _i]),
    "frhip_att_one_v4": (_i, [_i] + [_vp] * 12 + [_WP] * 4 + [_vp] * 7),
    "frhip_ffn_one": (_i, [_i, _i] + [_vp] * 6 + [_WP] * 3 + [_vp, _vp, _i, _vp, _vp]),
    "frhip_ffn_one_static": (_i, [_i, _i] + [_vp] * 6 + [_WP] * 3 + [_vp, _vp, _i, _vp]),
    "frhip_head": (_i, [_i, _vp, _vp, _vp, _WP, _vp, _vp]),
    "frhip_head_mirror": (_i, [_i, _vp, _vp, _vp, _WP, _vp, _vp, _vp]),
    "frhip_att_one_v5_1": (_i, [_i, _i] + [_vp] * 13 + [_WP] * 5 + [_vp] * 5),
    "frhip_att_one_v5": (_i, [_i, _i] + [_vp] * 12 + [_WP] * 4 + [_vp] * 5),
    "frhip_argmax_f32": (_i, [_vp, _i, _vp, _vp]),
    "frhip_argmax_blocks_f32": (_i, [_vp, _i, _vp, _i, _vp]),
    "frhip_argmax_blocks_f32_mirror": (_i, [_vp, _i, _vp, _vp, _i, _vp]),
    "frhip_gemm": (_i, [_vp, _WP, _vp, _i, _i, _vp]),
    "frhip_gemm_act": (_i, [_vp, _WP, _vp, _i, _i, _vp]),
    "frhip_copy_probe": (_i, [_vp, _vp, _sz, _vp]),
    "frhip_read_probe": (_i, [_vp, _sz, _vp, _vp]),
    "frhip_mfma_probe": (_i, [_i, _i, _vp, _vp, _vp, _vp]),
    "frhip_seq_workspace_bytes": (_sz, [_i, _i, _i]),
    "frhip_ffn_seq": (_i, [_i, _i, _i] + [_vp] * 6 + [_WP] * 3 + [_vp, _vp, _i, _vp, _vp]),
    "frhip_att_seq_v4": (_i, [_i, _i] + [_vp] * 12 + [_WP] * 4 + [_vp] * 7),
    "frhip_att_seq_v5_2": (_i, [_i, _i, _i] + [_vp] * 13 + [_WP] * 5 + [_vp] * 5),
    "frhip_att_seq_v5": (_i, [_i, _i, _i] + [_vp] * 12 + [_WP] * 4 + [_vp] * 5),
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


# --------------------------------------------------------------------------
# host layer (libfr_host.so): rwkv::Model through its C API
# --------------------------------------------------------------------------
_host = None


def host():
    global _host
    if _host is None:
        if not os.path.exists(LIBHOST):
            raise FrhipError("libfr_host.so is not built: run `python -c 'import __graft_entry__ as g; g.build()'`")
        lib()  # libfrhip.so first, so that the dependency resolves to the in-tree copy
        h = C.CDLL(LIBHOST)
        h.fr_last_error.restype = C.c_char_p
        h.fr_model_create.restype = _vp
        h.fr_model_create.argtypes = [C.c_char_p, C.c_char_p]
        h.fr_model_free.argtypes = [_vp]
        h.fr_model_info.argtypes = [_vp, C.POINTER(_i)]
        h.fr_model_run.argtypes = [_vp, _vp, _i, _vp, _i]
        h.fr_model_run_full.restype = C.c_longlong
        h.fr_model_run_full.argtypes = [_vp, _vp, _i, _vp, C.c_longlong]
        h.fr_sampler_create.restype = _vp
        h.fr_sampler_create.argtypes = [_i, _i]
        h.fr_sampler_free.argtypes = [_vp]
        h.fr_sampler_set_seed.argtypes = [_vp, _i]
        h.fr_sampler_sample.argtypes = [_vp, _vp, _i, C.c_float, _i, C.c_float]
        h.fr_sample_decode.restype = C.c_longlong
        h.fr_sample_decode.argtypes = [_vp, _vp, _i, _i, C.c_float, _i, C.c_float, _vp]
        h.fr_chat_decode.restype = C.c_longlong
        h.fr_chat_decode.argtypes = [_vp, _vp, _i, _i, C.c_float, _i, C.c_float, C.c_float, C.c_float, C.c_float, _vp]
        h.fr_model_reset.argtypes = [_vp]
        h.fr_model_save_state.argtypes = [_vp, C.c_char_p]
        h.fr_model_load_state.argtypes = [_vp, C.c_char_p]
        h.fr_model_get_state.argtypes = [_vp, _i, _i, _vp, _i]
        h.fr_model_set_state.argtypes = [_vp, _i, _i, _vp, _i]
        h.fr_model_snapshot.restype = _vp
        h.fr_model_snapshot.argtypes = [_vp]
        h.fr_model_restore.argtypes = [_vp, _vp]
        h.fr_snapshot_free.argtypes = [_vp]
        h.fr_greedy_decode.restype = C.c_longlong
        h.fr_greedy_decode.argtypes = [_vp, _i, _i, _vp]
        h.fr_quantize_u8.argtypes = [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp]
        h.fr_allocator_stats.argtypes = [C.POINTER(_sz)] * 3
        h.fr_allocator_trim.restype = C.c_longlong
        h.fr_hip_alloc.restype = _vp
        h.fr_hip_alloc.argtypes = [_sz]
        h.fr_hip_free.argtypes = [_vp]
        h.fr_hip_shape_op.restype = C.c_longlong
        h.fr_hip_shape_op.argtypes = [_i, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, C.c_longlong, _vp, _vp]
        _host = h
    return _host


def allocator_stats():
    """(bytes reserved from the driver, bytes handed out, driver allocation calls so far) of the hip allocator."""
    a, b, c = _sz(), _sz(), _sz()
    if host().fr_allocator_stats(C.byref(a), C.byref(b), C.byref(c)) < 0:
        raise FrhipError(host().fr_last_error().decode())
    return a.value, b.value, c.value


def shape_op(op, a, b=None, params=()):
    """One registry call of slice (op 0), cat (1), transpose (2) or silu (3) on the hip device."""
    a = np.ascontiguousarray(a)
    code = {np.dtype(np.float32): 0, np.dtype(np.float16): 1, np.dtype(np.int8): 2}[a.dtype]
    ash = (C.c_int * a.ndim)(*a.shape)
    bsh = None
    if b is not None:
        b = np.ascontiguousarray(b, a.dtype)
        bsh = (C.c_int * b.ndim)(*b.shape)
    par = (C.c_int * max(len(params), 1))(*params)
    out = np.empty(a.size + (b.size if b is not None else 0), a.dtype)
    osh, ond = (C.c_int * 4)(), C.c_int()
    n = host().fr_hip_shape_op(op, code, a.ctypes.data, ash, a.ndim, b.ctypes.data if b is not None else None, bsh, par,
                               out.ctypes.data, out.nbytes, osh, C.byref(ond))
    if n < 0:
        raise FrhipError(host().fr_last_error().decode())
    return out[:n].reshape([osh[i] for i in range(ond.value)])


class Model:
    """rwkv::Model(path, strategy) -- strategy "hip fp16" or "hip int8"; path a .fr file or
    "synthetic:v=4,L=..,C=..,F=..,V=..,seed=.."."""

    def __init__(self, path, strategy):
        self._h = host()
        self._m = self._h.fr_model_create(path.encode(), strategy.encode())
        if not self._m:
            raise FrhipError("Model(%r, %r): %s" % (path, strategy, self._h.fr_last_error().decode()))
        info = (_i * 6)()
        self._chk(self._h.fr_model_info(self._m, info))
        self.n_layer, self.n_embd, self.n_att, self.n_ffn, self.n_head, self.vocab = list(info)
        self._logits = np.empty(1 << 20, np.float32)

    def _chk(self, rc):
        if rc < 0:
            raise FrhipError(self._h.fr_last_error().decode())
        return rc

    def run(self, ids):
        """Model::Run: an int runs one token, a sequence runs seq mode; returns fp32 logits."""
        ids = np.atleast_1d(np.asarray(ids, np.int32))
        n = self._chk(self._h.fr_model_run(self._m, ids.ctypes.data, len(ids), self._logits.ctypes.data,
                                           self._logits.size))
        return self._logits[:n].copy()

    def run_full(self, ids):
        """ModelForwardSeq(..., full_output=true): fp32 logits of every position, [T, vocab]."""
        ids = np.ascontiguousarray(ids, np.int32)
        out = np.empty((len(ids), self._logits.size), np.float32)
        n = self._chk(self._h.fr_model_run_full(self._m, ids.ctypes.data, len(ids), out.ctypes.data, out.size))
        return out.reshape(-1)[:n].reshape(len(ids), -1)

    def reset(self):
        self._chk(self._h.fr_model_reset(self._m))

    # The names of the reference's Python wrapper (python/fr_python.cpp:48-56, python/fasterrwkv/__init__.py:19-25):
    # model(ids) -> logits as a numpy array, model.reset_states(), model.states().
    __call__ = run
    reset_states = reset

    def states(self):
        """Model::states() copied to the host: per layer a list of numpy arrays (RWKV-4: [C] act, three [C] fp32,
        [C] act; RWKV-5.x: [C] act, [H, S, S] fp32, [C] act -- model.cpp:145-177)."""
        v5 = self.n_head > 0  # RWKV-4 models have no heads
        out = []
        for l in range(self.n_layer):
            if v5:
                S = self.n_embd // self.n_head
                out.append([self.state(l, 0, np.float16), self.state(l, 1, np.float32).reshape(self.n_head, S, S),
                            self.state(l, 2, np.float16)])
            else:
                out.append([self.state(l, 0, np.float16)] + [self.state(l, j, np.float32) for j in (1, 2, 3)]
                           + [self.state(l, 4, np.float16)])
        return out

    def save_state(self, path):
        self._chk(self._h.fr_model_save_state(self._m, path.encode()))

    def load_state(self, path):
        self._chk(self._h.fr_model_load_state(self._m, path.encode()))

    def state(self, layer, index, dtype):
        buf = np.empty(1 << 22, np.uint8)
        n = self._chk(self._h.fr_model_get_state(self._m, layer, index, buf.ctypes.data, buf.size))
        return buf[:n].view(dtype).copy()

    def set_state(self, layer, index, a):
        """Replace one state tensor by a numpy array of the same size and dtype (what LoadStateFile does per tensor)."""
        a = np.ascontiguousarray(a)
        self._chk(self._h.fr_model_set_state(self._m, layer, index, a.ctypes.data, a.nbytes))

    def snapshot(self):
        """A copy of Model::states() (shares storage, as `auto s = model.states();` does); give it to restore()."""
        s = self._h.fr_model_snapshot(self._m)
        if not s:
            raise FrhipError(self._h.fr_last_error().decode())
        return s

    def restore(self, snap):
        """Model::set_states(snapshot)."""
        self._chk(self._h.fr_model_restore(self._m, snap))

    def free_snapshot(self, snap):
        self._h.fr_snapshot_free(snap)

    def generate(self, sampler, first_id, steps, temperature=1.0, top_k=0, top_p=1.0, presence_penalty=0.0,
                 frequency_penalty=0.0, penalty_decay=1.0):
        """The generation loop of chat.cpp:56-92 in C++ (its penalties are 0.8, 0.8 and 0.996, chat.cpp:22-24);
        returns (token ids, seconds)."""
        out = np.empty(steps, np.int32)
        if presence_penalty or frequency_penalty:
            us = self._h.fr_chat_decode(self._m, sampler._s, int(first_id), int(steps), temperature, top_k, top_p,
                                        presence_penalty, frequency_penalty, penalty_decay, out.ctypes.data)
        else:
            us = self._h.fr_sample_decode(self._m, sampler._s, int(first_id), int(steps), temperature, top_k, top_p,
                                          out.ctypes.data)
        if us < 0:
            raise FrhipError(self._h.fr_last_error().decode())
        return out, us * 1e-6

    def greedy(self, first_id, steps):
        """chat.cpp's greedy loop in C++; returns (token ids, seconds)."""
        out = np.empty(steps, np.int32)
        us = self._h.fr_greedy_decode(self._m, int(first_id), int(steps), out.ctypes.data)
        if us < 0:
            raise FrhipError(self._h.fr_last_error().decode())
        return out, us * 1e-6

    def close(self):
        if getattr(self, "_m", None):
            self._h.fr_model_free(self._m)
            self._m = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Sampler:
    """rwkv::Sampler (sampler.h:8-16): temperature / top-k / top-p sampling on host logits with a
    std::minstd_rand0 stream; `seed=None` seeds from the random device as the reference does."""

    def __init__(self, seed=None):
        self._h = host()
        self._s = self._h.fr_sampler_create(0 if seed is None else int(seed), 0 if seed is None else 1)
        if not self._s:
            raise FrhipError(self._h.fr_last_error().decode())

    def set_seed(self, seed):
        self._h.fr_sampler_set_seed(self._s, int(seed))

    def sample(self, logits, temperature=1.0, top_k=0, top_p=1.0):
        x = np.ascontiguousarray(logits, np.float32)
        r = self._h.fr_sampler_sample(self._s, x.ctypes.data, x.size, temperature, top_k, top_p)
        if r < 0:
            raise FrhipError(self._h.fr_last_error().decode())
        return r

    __call__ = sample  # python/fasterrwkv/__init__.py:25

    def __del__(self):
        if getattr(self, "_s", None):
            self._h.fr_sampler_free(self._s)
            self._s = None


def write_fr(path, version, n_layer, n_embd, n_ffn, n_head, params, emb, quantized=None):
    """Write a `.fr` file (msgpack layout of tools/convert_weight.py:12-55) from numpy arrays in
    the positional parameter order.  `quantized` maps a parameter index to (q, mx, rx, my, ry)."""
    import msgpack
    names = []
    for l in range(n_layer):
        b, a, f = "blocks.%d." % l, "blocks.%d.att." % l, "blocks.%d.ffn." % l
        names += [b + "ln1.weight", b + "ln1.bias"]
        if version != "4":
            names += [a + "ln_x.weight", a + "ln_x.bias"]
        names += [a + "time_mix_k", a + "time_mix_v", a + "time_mix_r"]
        if version in ("5.1", "5.2"):
            names += [a + "time_mix_g"]
        names += [a + "time_decay", a + "time_first", a + "key.weight", a + "value.weight", a + "receptance.weight"]
        if version in ("5.1", "5.2"):
            names += [a + "gate.weight"]
        names += [a + "output.weight", b + "ln2.weight", b + "ln2.bias", f + "time_mix_k", f + "time_mix_r",
                  f + "key.weight", f + "value.weight", f + "receptance.weight"]
    names += ["ln_out.weight", "ln_out.bias", "head.weight"]
    assert len(names) == len(params), (len(names), len(params))
    tname = {np.dtype(np.float16): "torch.float16", np.dtype(np.float32): "torch.float32",
             np.dtype(np.uint8): "torch.uint8"}

    def pack(a):
        a = np.ascontiguousarray(a)
        return {"dtype": tname[a.dtype], "data": a.tobytes(), "shape": list(a.shape)}

    weights = {}
    for i, (n, p) in enumerate(zip(names, params)):
        if quantized and i in quantized:
            q, mx, rx, my, ry = quantized[i]
            weights[n] = pack(q)
            for suf, v in (("_mx", mx), ("_rx", rx), ("_my", my), ("_ry", ry)):
                weights[n + suf] = pack(np.asarray(v, np.float16))
        else:
            weights[n] = pack(p)
    d = {"embd_weights": [pack(r) for r in emb], "weights": weights, "version": version, "n_layer": n_layer,
         "n_embd": n_embd, "n_att": n_embd, "n_ffn": n_ffn}
    if version != "4":
        d["n_head"] = n_head
    with open(path, "wb") as fh:
        msgpack.pack(d, fh, use_bin_type=True)
