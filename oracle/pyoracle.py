"""ctypes binding of the CPU oracle (oracle/librwkv_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py -- never by the shipped package.

Arrays cross the boundary as numpy arrays: binary16 data as np.float16 (or
np.uint16 bit patterns), fp32 as np.float32, uint8 codes as np.uint8.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "librwkv_oracle.so")

F32, F16 = 0, 1


def build(force=False):
    """Compile the oracle with gcc (oracle/Makefile)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


lib = _load()

_vp = C.c_void_p
_i = C.c_int


def _p(a):
    if a is None:
        return None
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"], "need a contiguous numpy array"
    return a.ctypes.data_as(_vp)


def _sig(name, res, *args):
    f = getattr(lib, name)
    f.restype = res
    f.argtypes = list(args)
    return f


_sig("orc_f2h", C.c_uint16, C.c_float)
_sig("orc_h2f", C.c_float, C.c_uint16)
_sig("orc_d2h", C.c_uint16, C.c_double)
for _n in ("orc_hadd", "orc_hsub", "orc_hmul", "orc_hdiv"):
    _sig(_n, C.c_uint16, C.c_uint16, C.c_uint16)
_sig("orc_hfma", C.c_uint16, C.c_uint16, C.c_uint16, C.c_uint16)
_sig("orc_f2h_n", None, _vp, _vp, C.c_size_t)
_sig("orc_h2f_n", None, _vp, _vp, C.c_size_t)
_sig("orc_layernorm_f16", None, _vp, _vp, _vp, _vp, _i, _i)
_sig("orc_layernorm_f32", None, _vp, _vp, _vp, _vp, _i, _i)
_sig("orc_groupnorm_f32", None, _vp, _i, _vp, _vp, _vp, _i, _i)
_sig("orc_mix_f16", None, _vp, _vp, _vp, _vp, _i, _i)
_sig("orc_gemm_f16", None, _vp, _vp, _vp, _vp, _i, _i, _i)
_sig("orc_gemm_f32", None, _vp, _vp, _vp, _i, _i, _i)
_sig("orc_sigmoid_f16", None, _vp, C.c_size_t)
_sig("orc_relu_square_f16", None, _vp, C.c_size_t)
_sig("orc_silu_f16", None, _vp, C.c_size_t)
_sig("orc_wkv4_one_f16", None, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i)
_sig("orc_dequant_u8_scalar", C.c_uint16, C.c_uint8, C.c_uint16, C.c_uint16, C.c_uint16, C.c_uint16)
_sig("orc_dequant_u8", None, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i)
_sig("orc_att_one_v4_f16", None, *([_vp] * 18), _i)
_sig("orc_att_seq_v4_f16", None, *([_vp] * 18), _i, _i)
_sig("orc_ffn_one_f16", None, *([_vp] * 11), _i, _i)
_sig("orc_ffn_seq_f16", None, *([_vp] * 11), _i, _i, _i)
_sig("orc_att_one_v5_1_f16", None, *([_vp] * 20), _i, _i)
_sig("orc_att_seq_v5_2_f16", None, *([_vp] * 20), _i, _i, _i)
_sig("orc_wkv5_2_seq_f32", None, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i)
_sig("orc_att_one_v5_f16", None, *([_vp] * 18), _i, _i)
_sig("orc_att_seq_v5_f16", None, *([_vp] * 18), _i, _i, _i)
_sig("orc_wkv5_seq_matrix_f32", None, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i)
_sig("orc_argmax", _i, _vp, _i)


# --------------------------------------------------------------------------
# primitive wrappers (allocate outputs, return numpy)
# --------------------------------------------------------------------------
def f2h(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.float16)
    lib.orc_f2h_n(_p(x), _p(out), x.size)
    return out


def h2f(x):
    x = np.ascontiguousarray(x, dtype=np.float16)
    out = np.empty(x.shape, dtype=np.float32)
    lib.orc_h2f_n(_p(x), _p(out), x.size)
    return out


def layernorm_f16(x, g, b):
    x = np.ascontiguousarray(x, np.float16)
    rows, cols = (1, x.shape[0]) if x.ndim == 1 else x.shape
    y = np.empty_like(x)
    lib.orc_layernorm_f16(_p(x), _p(g), _p(b), _p(y), rows, cols)
    return y


def layernorm_f32(x, g, b):
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = (1, x.shape[0]) if x.ndim == 1 else x.shape
    y = np.empty_like(x)
    lib.orc_layernorm_f32(_p(x), _p(g), _p(b), _p(y), rows, cols)
    return y


def groupnorm_f32(x, groups, g, b):
    x = np.ascontiguousarray(x, np.float32)
    rows, cols = (1, x.shape[0]) if x.ndim == 1 else x.shape
    y = np.empty_like(x)
    lib.orc_groupnorm_f32(_p(x), groups, _p(g), _p(b), _p(y), rows, cols)
    return y


def mix_f16(xx, sx, m):
    xx = np.ascontiguousarray(xx, np.float16)
    rows, cols = (1, xx.shape[0]) if xx.ndim == 1 else xx.shape
    out = np.empty_like(xx)
    lib.orc_mix_f16(_p(xx), _p(np.ascontiguousarray(sx, np.float16)), _p(m), _p(out), rows, cols)
    return out


def gemm_f16(x, W, out="f32"):
    """x [T,K] or [K] half, W [K,N] half -> fp32 accumulate, rounded once to `out`."""
    x = np.ascontiguousarray(x, np.float16)
    W = np.ascontiguousarray(W, np.float16)
    T = 1 if x.ndim == 1 else x.shape[0]
    K, N = W.shape
    shape = (N,) if x.ndim == 1 else (T, N)
    if out == "f32":
        y = np.empty(shape, np.float32)
        lib.orc_gemm_f16(_p(x), _p(W), _p(y), None, T, K, N)
    else:
        y = np.empty(shape, np.float16)
        lib.orc_gemm_f16(_p(x), _p(W), None, _p(y), T, K, N)
    return y


def gemm_f32(x, W):
    x = np.ascontiguousarray(x, np.float32)
    W = np.ascontiguousarray(W, np.float32)
    T = 1 if x.ndim == 1 else x.shape[0]
    K, N = W.shape
    y = np.empty((N,) if x.ndim == 1 else (T, N), np.float32)
    lib.orc_gemm_f32(_p(x), _p(W), _p(y), T, K, N)
    return y


def sigmoid_f16(x):
    y = np.array(x, dtype=np.float16, copy=True)
    lib.orc_sigmoid_f16(_p(y), y.size)
    return y


def relu_square_f16(x):
    y = np.array(x, dtype=np.float16, copy=True)
    lib.orc_relu_square_f16(_p(y), y.size)
    return y


def silu_f16(x):
    y = np.array(x, dtype=np.float16, copy=True)
    lib.orc_silu_f16(_p(y), y.size)
    return y


def wkv4_one_f16(t_first, t_decay, k, v, aa, bb, pp, r):
    """Returns (r_out, aa', bb', pp'); inputs untouched."""
    aa, bb, pp = aa.copy(), bb.copy(), pp.copy()
    r = np.array(r, dtype=np.float16, copy=True)
    lib.orc_wkv4_one_f16(_p(t_first), _p(t_decay), _p(k), _p(v), _p(aa), _p(bb), _p(pp), _p(r), r.size)
    return r, aa, bb, pp


_sig("orc_gemv_u8", None, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i)
_sig("orc_register_u8", None, _vp, _vp, _vp, _vp, _vp, _vp)
_sig("orc_unregister_u8", None, _vp)


def gemv_u8(x, q, mx, rx, my, ry):
    """One-token product on the unrounded fp32 weights of the codes: x [K] half -> y [N] fp32."""
    K, N = q.shape
    y = np.empty(N, np.float32)
    lib.orc_gemv_u8(_p(np.ascontiguousarray(x, np.float16)), _p(q), _p(mx), _p(rx), _p(my), _p(ry), _p(y), K, N)
    return y


ACC_EXACT, ACC_F32_SEQUENTIAL = 0, 1
_sig("orc_set_accumulation", None, _i)


def set_accumulation(mode):
    """ACC_EXACT (default): products accumulate exactly, one rounding to fp32; ACC_F32_SEQUENTIAL: fp32 in
    ascending k -- another valid member of the reference's "fp32 accumulate in cuBLAS's order"."""
    lib.orc_set_accumulation(int(mode))


_u8_keep = {}


def register_u8(W, q, mx, rx, my, ry):
    """From now on the oracle's one-token products on the binary16 matrix W (= dequant_u8 of these
    codes) multiply the unrounded fp32 weights of the codes (orc_gemv_u8); matrix x matrix products
    keep multiplying W.  The arrays are held until unregister_u8(W)."""
    assert isinstance(W, np.ndarray) and W.dtype == np.float16 and W.flags["C_CONTIGUOUS"] and W.shape == q.shape
    parts = [np.ascontiguousarray(q, np.uint8)] + [np.ascontiguousarray(v, np.float16) for v in (mx, rx, my, ry)]
    _u8_keep[W.ctypes.data] = (W, parts)
    lib.orc_register_u8(_p(W), *[_p(a) for a in parts])
    return W


def unregister_u8(W):
    if _u8_keep.pop(W.ctypes.data, None) is not None:
        lib.orc_unregister_u8(_p(W))


def dequant_u8(q, mx, rx, my, ry):
    """q [K,N] uint8, mx/rx [N], my/ry [K] half -> W^ [K,N] half."""
    K, N = q.shape
    W = np.empty((K, N), np.float16)
    lib.orc_dequant_u8(_p(q), _p(mx), _p(rx), _p(my), _p(ry), _p(W), K, N)
    return W


def att_one_v4_f16(x, sx, aa, bb, pp, ln_w, ln_b, mk, mv, mr, td, tf, kw, vw, rw, ow):
    """kernels/cuda/att.cu:337-359 -> (x_out, xx, aa', bb', pp')."""
    C_ = x.shape[-1]
    T = 1 if x.ndim == 1 else x.shape[0]
    aa, bb, pp = aa.copy(), bb.copy(), pp.copy()
    x_out = np.empty_like(x)
    xx = np.empty(C_, np.float16)
    lib.orc_att_seq_v4_f16(_p(x), _p(sx), _p(aa), _p(bb), _p(pp), _p(ln_w), _p(ln_b), _p(mk), _p(mv),
                           _p(mr), _p(td), _p(tf), _p(kw), _p(vw), _p(rw), _p(ow), _p(x_out), _p(xx),
                           T, C_)
    return x_out, xx, aa, bb, pp


att_seq_v4_f16 = att_one_v4_f16


def ffn_f16(x, sx, ln_w, ln_b, mk, mr, kw, vw, rw):
    """kernels/cuda/ffn.cu:89-110 / ffn_seq.cu:89-109 -> (x_out, xx_last)."""
    C_ = x.shape[-1]
    T = 1 if x.ndim == 1 else x.shape[0]
    F_ = kw.shape[1]
    x_out = np.empty_like(x)
    xx = np.empty(C_, np.float16)
    lib.orc_ffn_seq_f16(_p(x), _p(sx), _p(ln_w), _p(ln_b), _p(mk), _p(mr), _p(kw), _p(vw), _p(rw),
                        _p(x_out), _p(xx), T, C_, F_)
    return x_out, xx


def att_v5_2_f16(x, sx, s, ln_w, ln_b, lx_w, lx_b, mk, mv, mr, mg, td, tf, kw, vw, rw, gw, ow, H):
    """One token (x.ndim==1: att.cu:393-425) or sequence (att_seq.cu:464-493)
    -> (x_out, xx_last, s')."""
    C_ = x.shape[-1]
    s = s.copy()
    x_out = np.empty_like(x)
    xx = np.empty(C_, np.float16)
    args = [_p(a) for a in (x, sx, s, ln_w, ln_b, lx_w, lx_b, mk, mv, mr, mg, td, tf, kw, vw, rw, gw,
                            ow, x_out, xx)]
    if x.ndim == 1:
        lib.orc_att_one_v5_1_f16(*args, C_, H)
    else:
        lib.orc_att_seq_v5_2_f16(*args, x.shape[0], C_, H)
    return x_out, xx, s


def att_v5_0_f16(x, sx, s, ln_w, ln_b, lx_w, lx_b, mk, mv, mr, td, tf, kw, vw, rw, ow, H):
    """RWKV-5.0.  One token (x.ndim==1: att.cu:362-391) or sequence in matrix form
    (att_seq.cu:425-462) -> (x_out, xx_last, s')."""
    C_ = x.shape[-1]
    s = s.copy()
    x_out = np.empty_like(x)
    xx = np.empty(C_, np.float16)
    args = [_p(a) for a in (x, sx, s, ln_w, ln_b, lx_w, lx_b, mk, mv, mr, td, tf, kw, vw, rw, ow, x_out, xx)]
    if x.ndim == 1:
        lib.orc_att_one_v5_f16(*args, C_, H)
    else:
        lib.orc_att_seq_v5_f16(*args, x.shape[0], C_, H)
    return x_out, xx, s


def wkv5_seq_matrix_f32(s, r, k, v, w, u):
    """att_seq.cu:181-243 (RWKV-5.0 matrix form); w, u [H]."""
    T, C_ = r.shape
    H = w.shape[0]
    s = s.copy()
    y = np.empty((T, C_), np.float32)
    lib.orc_wkv5_seq_matrix_f32(_p(s), _p(r), _p(k), _p(v), _p(w), _p(u), _p(y), T, H, C_ // H)
    return y, s


def wkv5_2_seq_f32(s, r, k, v, w, u):
    T, C_ = r.shape
    H, S = w.shape
    s = s.copy()
    y = np.empty((T, C_), np.float32)
    lib.orc_wkv5_2_seq_f32(_p(s), _p(r), _p(k), _p(v), _p(w), _p(u), _p(y), T, H, S)
    return y, s


# --------------------------------------------------------------------------
# whole model
# --------------------------------------------------------------------------
class _OrcModel(C.Structure):
    _fields_ = [("version", _i), ("mode", _i), ("n_layer", _i), ("n_embd", _i), ("n_att", _i),
                ("n_ffn", _i), ("n_head", _i), ("vocab", _i), ("params", C.POINTER(_vp)),
                ("emb", _vp)]


_sig("orc_state_count", C.c_size_t, C.POINTER(_OrcModel))
_sig("orc_state_elems", C.c_size_t, C.POINTER(_OrcModel), C.c_size_t)
_sig("orc_state_is_act", _i, C.POINTER(_OrcModel), C.c_size_t)
_sig("orc_state_reset", None, C.POINTER(_OrcModel), C.POINTER(_vp))
_sig("orc_model_forward", None, C.POINTER(_OrcModel), C.POINTER(_vp), _i, _vp)
_sig("orc_model_forward_seq", None, C.POINTER(_OrcModel), C.POINTER(_vp), _vp, _i, _vp)


class Model:
    """Oracle model over a list of numpy parameter arrays in the reference's
    positional order (kernels/default/init_model.cpp:91-126) plus emb [V,C]."""

    def __init__(self, version, mode, n_layer, n_embd, n_ffn, n_head, vocab, params, emb, n_att=None, quant=None):
        """quant: {parameter index: (q, mx, rx, my, ry)} -- that parameter becomes the binary16 matrix w^ of the
        codes (seq mode multiplies it) and one-token steps multiply the codes' unrounded fp32 weights."""
        self.mode = mode
        self._params = [np.ascontiguousarray(p) for p in params]
        self._registered = []
        for i, parts in (quant or {}).items():
            assert mode == F16
            self._params[i] = register_u8(dequant_u8(*parts), *parts)
            self._registered.append(self._params[i])
        self._emb = np.ascontiguousarray(emb)
        self._parr = (_vp * len(self._params))(*[_p(p) for p in self._params])
        self.c = _OrcModel(version, mode, n_layer, n_embd, n_att or n_embd, n_ffn, n_head, vocab,
                           C.cast(self._parr, C.POINTER(_vp)), _p(self._emb))
        self.vocab = vocab
        cnt = lib.orc_state_count(C.byref(self.c))
        act = np.float16 if mode == F16 else np.float32
        self.state = [np.zeros(lib.orc_state_elems(C.byref(self.c), i),
                               act if lib.orc_state_is_act(C.byref(self.c), i) else np.float32)
                      for i in range(cnt)]
        self._sarr = (_vp * cnt)(*[_p(s) for s in self.state])
        self.reset()

    def reset(self):
        lib.orc_state_reset(C.byref(self.c), self._sarr)

    def close(self):
        for w in getattr(self, "_registered", []):
            unregister_u8(w)
        self._registered = []

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def run(self, ids):
        """Model::Run (model.cpp:188-208): int -> one-token forward, list -> seq mode."""
        logits = np.empty(self.vocab, np.float32)
        if isinstance(ids, (int, np.integer)):
            lib.orc_model_forward(C.byref(self.c), self._sarr, int(ids), _p(logits))
        else:
            ids = np.ascontiguousarray(ids, np.int32)
            lib.orc_model_forward_seq(C.byref(self.c), self._sarr, _p(ids), len(ids), _p(logits))
        return logits
