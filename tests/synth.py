"""Synthetic RWKV weights for tests, in the reference's positional parameter order
(kernels/default/init_model.cpp:91-126).  Distributions follow the benchmark
configurations: 2-D weights ~N(0, 0.02); time_decay_raw ~U(-5,1) (v4) / U(-6,0)
(v5.2); time_first ~U(-1,1); time_mix ~U(0,1); layernorm gamma=1, beta=0 (tests
perturb gamma/beta slightly so that the affine part is exercised).
Stored forms are the ones the kernels consume: v4 time_decay = -exp(raw) (fp32);
v5.2 time_decay = exp(-exp(raw)) [H,S] (fp32), v5.0 (version=50) the same with one
value per head [H] and no gate; matrices [in,out].
"""
import numpy as np


def _ln_rows(e):
    m = e.mean(axis=1, keepdims=True)
    v = e.var(axis=1, keepdims=True)
    return (e - m) / np.sqrt(v + 1e-5)


def make_model(version, L, C, F, V, H=0, seed=0, dtype=np.float16, affine_jitter=0.05):
    """Returns (params list, emb [V,C]).  dtype is the weight/activation type."""
    rng = np.random.default_rng(seed)
    act = dtype

    def mat(k, n):
        return (rng.standard_normal((k, n), dtype=np.float32) * 0.02).astype(act)

    def ln():
        g = (1.0 + affine_jitter * rng.standard_normal(C)).astype(act)
        b = (affine_jitter * rng.standard_normal(C)).astype(act)
        return [g, b]

    def mixv():
        return rng.uniform(0, 1, C).astype(act)

    params = []
    for _ in range(L):
        params += ln()
        if version == 4:
            params += [mixv(), mixv(), mixv()]
            params += [(-np.exp(rng.uniform(-5, 1, C))).astype(np.float32),
                       rng.uniform(-1, 1, C).astype(np.float32)]
            params += [mat(C, C), mat(C, C), mat(C, C), mat(C, C)]
        elif version == 50:
            params += [(1.0 + affine_jitter * rng.standard_normal(C)).astype(np.float32),
                       (affine_jitter * rng.standard_normal(C)).astype(np.float32)]
            params += [mixv(), mixv(), mixv()]
            params += [np.exp(-np.exp(rng.uniform(-6, 0, H))).astype(np.float32),
                       rng.uniform(-1, 1, H).astype(np.float32)]
            params += [mat(C, C), mat(C, C), mat(C, C), mat(C, C)]
        else:
            S = C // H
            gx_t = np.float32 if True else act
            params += [(1.0 + affine_jitter * rng.standard_normal(C)).astype(gx_t),
                       (affine_jitter * rng.standard_normal(C)).astype(gx_t)]
            params += [mixv(), mixv(), mixv(), mixv()]
            params += [np.exp(-np.exp(rng.uniform(-6, 0, (H, S)))).astype(np.float32),
                       rng.uniform(-1, 1, (H, S)).astype(np.float32)]
            params += [mat(C, C), mat(C, C), mat(C, C), mat(C, C), mat(C, C)]
        params += ln()
        params += [mixv(), mixv()]
        params += [mat(C, F), mat(F, C), mat(C, C)]
    params += ln()
    params += [mat(C, V)]
    emb = _ln_rows(rng.standard_normal((V, C), dtype=np.float32) * 0.02).astype(act)
    if dtype == np.float32:
        params = [p.astype(np.float32) for p in params]
    return params, emb


def quantize_u8(w):
    """ChatRWKV-style uint8 weight-only quantisation of a [K,N] matrix:
    per-column minimum mx and range rx, per-row minimum my and range ry (binary16),
    q = clamp(round((w - my - mx) / (rx*ry) * 255), 0, 255).
    Returns (q uint8 [K,N], mx [N], rx [N], my [K], ry [K])."""
    w = np.asarray(w, np.float32)
    mx = w.min(axis=0).astype(np.float16)
    r = w - mx.astype(np.float32)[None, :]
    my = r.min(axis=1).astype(np.float16)
    r = r - my.astype(np.float32)[:, None]
    rx = np.maximum(r.max(axis=0), 1e-4).astype(np.float16)
    r = r / rx.astype(np.float32)[None, :]
    ry = np.maximum(r.max(axis=1), 1e-4).astype(np.float16)
    r = r / ry.astype(np.float32)[:, None]
    q = np.clip(np.rint(r * 255.0), 0, 255).astype(np.uint8)
    return q, mx, rx, my, ry


MATRIX_POS_V4 = (7, 8, 9, 10, 15, 16, 17)
MATRIX_POS_V50 = (9, 10, 11, 12, 17, 18, 19)
MATRIX_POS_V52 = (10, 11, 12, 13, 14, 19, 20, 21)


def matrix_indices(version, L):
    per = {4: 18, 50: 20}.get(version, 22)
    pos = {4: MATRIX_POS_V4, 50: MATRIX_POS_V50}.get(version, MATRIX_POS_V52)
    idx = [l * per + p for l in range(L) for p in pos]
    idx.append(L * per + 2)  # head.weight
    return idx
