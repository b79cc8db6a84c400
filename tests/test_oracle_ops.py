"""Pins each oracle function against something independent of its own formula:
library routines, float64 brute force, closed forms and special cases."""
import numpy as np
import pytest
import torch

import pyoracle as po
from synth import quantize_u8

rng = np.random.default_rng(7)


def h(x):
    return np.asarray(x, np.float32).astype(np.float16)


# ---------------------------------------------------------------- layernorm
def test_layernorm_f32_matches_torch():
    x = rng.standard_normal((5, 768)).astype(np.float32) * 3 + 1
    g = rng.standard_normal(768).astype(np.float32)
    b = rng.standard_normal(768).astype(np.float32)
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x), (768,), torch.from_numpy(g),
                                         torch.from_numpy(b), 1e-5).numpy()
    assert np.allclose(po.layernorm_f32(x, g, b), ref, atol=2e-6, rtol=1e-5)


def test_layernorm_f16_rounding_points():
    """normalise in fp32 -> half -> *gamma in half -> +beta in half
    (kernels/cuda/layer_norm.cu:60-69)."""
    x = h(rng.standard_normal((3, 2048)) * 2)
    g = h(1 + 0.1 * rng.standard_normal(2048))
    b = h(0.1 * rng.standard_normal(2048))
    xf = x.astype(np.float64)
    mean = xf.mean(axis=1, keepdims=True)
    var = xf.var(axis=1, keepdims=True)
    n = ((xf - mean) / np.sqrt(var + 1e-5)).astype(np.float32).astype(np.float16)
    ref = ((n * g).astype(np.float16) + b).astype(np.float16)
    got = po.layernorm_f16(x, g, b)
    # the fp32 normalised value can sit next to a half rounding boundary: allow 1 ulp on a few
    diff = np.abs(got.view(np.int16).astype(np.int32) - ref.view(np.int16).astype(np.int32))
    assert diff.max() <= 1 and (diff > 0).mean() < 0.01


def test_layernorm_special_cases():
    C = 512
    g = h(rng.standard_normal(C))
    b = h(rng.standard_normal(C))
    const = np.full(C, 3.25, np.float16)
    assert np.array_equal(po.layernorm_f16(const, g, b), b)  # zero variance -> beta
    x = h(rng.standard_normal(C))
    y = po.layernorm_f16(x, np.ones(C, np.float16), np.zeros(C, np.float16)).astype(np.float64)
    assert abs(y.mean()) < 2e-3 and abs(y.var() - 1) < 5e-3


def test_groupnorm_matches_torch():
    H, S, T = 40, 64, 3
    x = rng.standard_normal((T, H * S)).astype(np.float32) * 2
    g = rng.standard_normal(H * S).astype(np.float32)
    b = rng.standard_normal(H * S).astype(np.float32)
    ref = torch.nn.functional.group_norm(torch.from_numpy(x), H, torch.from_numpy(g),
                                         torch.from_numpy(b), 1e-5).numpy()
    assert np.allclose(po.groupnorm_f32(x, H, g, b), ref, atol=3e-6, rtol=1e-5)


# ---------------------------------------------------------------------- mix
def test_mix_closed_form_and_limits():
    C = 1024
    xx, sx = h(rng.standard_normal(C)), h(rng.standard_normal(C))
    assert np.array_equal(po.mix_f16(xx, sx, np.ones(C, np.float16)), xx)   # m=1 -> xx
    assert np.array_equal(po.mix_f16(xx, sx, np.zeros(C, np.float16)), sx)  # m=0 -> sx
    m = h(rng.uniform(0, 1, C))
    ref = ((xx * m).astype(np.float16) + (sx * (np.float16(1) - m).astype(np.float16)).astype(np.float16))
    assert np.array_equal(po.mix_f16(xx, sx, m), ref.astype(np.float16))
    # broadcast of the mix vector over rows (att_seq.cu:34-36: mix[i % C])
    X, Sx = h(rng.standard_normal((4, C))), h(rng.standard_normal((4, C)))
    got = po.mix_f16(X, Sx, m)
    for t in range(4):
        assert np.array_equal(got[t], po.mix_f16(X[t], Sx[t], m))


# --------------------------------------------------------------------- gemm
@pytest.mark.parametrize("T,K,N", [(1, 2048, 512), (3, 300, 70), (9, 64, 257)])
def test_gemm_f16_against_float64(T, K, N):
    x = h(rng.standard_normal((T, K)))
    W = h(rng.standard_normal((K, N)) * 0.02)
    ref = x.astype(np.float64) @ W.astype(np.float64)
    got = po.gemm_f16(x, W, "f32")
    assert np.allclose(got, ref, atol=1e-5 * np.sqrt(K), rtol=1e-5)
    got16 = po.gemm_f16(x, W, "f16")
    assert np.array_equal(got16, got.astype(np.float16))  # one rounding of the fp32 sum
    if T == 1:
        assert np.array_equal(po.gemm_f16(x[0], W, "f32"), got[0])
    # a transposed-operand mistake would fail this asymmetric case
    e = np.zeros((1, K), np.float16)
    e[0, 5] = 1
    assert np.array_equal(po.gemm_f16(e, W, "f16")[0], W[5])


def test_gemm_f32_against_float64():
    x = rng.standard_normal((2, 333)).astype(np.float32)
    W = rng.standard_normal((333, 129)).astype(np.float32)
    assert np.allclose(po.gemm_f32(x, W), x.astype(np.float64) @ W.astype(np.float64), atol=1e-4)


# -------------------------------------------------------------- elementwise
def test_sigmoid_relu2_silu_closed_forms():
    x = h(np.linspace(-12, 12, 4001))
    xd = x.astype(np.float64)
    s = po.sigmoid_f16(x)
    ref = (1 / (1 + np.exp(-xd))).astype(np.float32).astype(np.float16)
    assert np.array_equal(s, ref)
    assert po.sigmoid_f16(h([0.0]))[0] == np.float16(0.5)
    r2 = po.relu_square_f16(x)
    assert np.array_equal(r2, np.where(xd > 0, (x * x).astype(np.float16), np.float16(0)))
    assert np.isinf(po.relu_square_f16(h([256.0]))[0])  # overflow above |x|>255.9 (ffn.cu:42-49)
    si = po.silu_f16(x)
    e = np.exp(-x.astype(np.float32)).astype(np.float16)
    ref = (x.astype(np.float32) / (np.float16(1) + e).astype(np.float16).astype(np.float32)).astype(np.float16)
    dif = np.abs(si.view(np.int16).astype(int) - ref.view(np.int16).astype(int))
    assert dif.max() <= 1  # expf vs numpy exp may differ in the last fp32 bit
    assert np.allclose(si.astype(np.float64), xd / (1 + np.exp(-xd)), rtol=3e-3, atol=1e-3)


def test_known_answer_one_half():
    """tests/test_ops.cpp:9-16: fill_(1); scalar_div_(2) == 0.5 in fp16."""
    one, two = 0x3C00, 0x4000
    assert po.lib.orc_hdiv(one, two) == np.float16(0.5).view(np.uint16)


# ---------------------------------------------------------------------- WKV
def _wkv4_closed_form(k, v, w, u):
    """wkv_t = (sum_{i<t} e^{(t-1-i)w + k_i} v_i + e^{u+k_t} v_t) / (same without v), float64."""
    T, C = k.shape
    out = np.zeros((T, C))
    for t in range(T):
        num = np.exp(u + k[t]) * v[t]
        den = np.exp(u + k[t])
        for i in range(t):
            e = np.exp((t - 1 - i) * w + k[i])
            num += e * v[i]
            den += e
        out[t] = num / den
    return out


def test_wkv4_recurrence_matches_closed_form_and_first_step_is_v():
    T, C = 12, 64
    k = rng.standard_normal((T, C)).astype(np.float32)
    v = rng.standard_normal((T, C)).astype(np.float32)
    w = (-np.exp(rng.uniform(-5, 1, C))).astype(np.float32)
    u = rng.uniform(-1, 1, C).astype(np.float32)
    ref = _wkv4_closed_form(k.astype(np.float64), v.astype(np.float64), w.astype(np.float64),
                            u.astype(np.float64))
    aa, bb = np.zeros(C, np.float32), np.zeros(C, np.float32)
    pp = np.full(C, -1e30, np.float32)
    for t in range(T):
        r, aa, bb, pp = po.wkv4_one_f16(u, w, k[t], v[t], aa, bb, pp, np.ones(C, np.float16))
        # r = h(1 * h(wkv)) = h(wkv)
        assert np.allclose(r.astype(np.float64), ref[t], rtol=2e-3, atol=2e-3), t
        if t == 0:
            assert np.array_equal(r, v[0].astype(np.float16))  # empty state: wkv_0 = v_0
    # the state after T steps, in shift-free form, equals the direct sums
    num = sum(np.exp((T - 1 - i) * w.astype(np.float64) + k[i]) * v[i] for i in range(T))
    den = sum(np.exp((T - 1 - i) * w.astype(np.float64) + k[i]) for i in range(T))
    assert np.allclose(aa * np.exp(pp.astype(np.float64)), num, rtol=1e-4)
    assert np.allclose(bb * np.exp(pp.astype(np.float64)), den, rtol=1e-4)


def test_wkv4_independent_of_max_shift():
    C = 32
    k, v = rng.standard_normal(C).astype(np.float32), rng.standard_normal(C).astype(np.float32)
    w = (-np.exp(rng.uniform(-5, 1, C))).astype(np.float32)
    u = rng.uniform(-1, 1, C).astype(np.float32)
    aa, bb = rng.uniform(0.5, 2, C).astype(np.float32), rng.uniform(0.5, 2, C).astype(np.float32)
    pp = rng.standard_normal(C).astype(np.float32)
    one = np.ones(C, np.float16)
    r1, a1, b1, p1 = po.wkv4_one_f16(u, w, k, v, aa, bb, pp, one)
    d = np.float32(1.5)  # the same state written with another exponent offset
    r2, a2, b2, p2 = po.wkv4_one_f16(u, w, k, v, aa * np.exp(d), bb * np.exp(d), pp - d, one)
    assert np.abs(r1.astype(np.float32) - r2.astype(np.float32)).max() <= 2e-3
    assert np.allclose(a1 * np.exp(p1.astype(np.float64)), a2 * np.exp(p2.astype(np.float64)), rtol=1e-4)


def _wkv5_brute(r, k, v, w, u, s0):
    """y_t = r_t . (diag(u) k_t v_t^T + S_{t-1});  S_t = diag(w) S_{t-1} + k_t v_t^T, float64,
    S indexed [head][key][value]."""
    T, C = r.shape
    H, S = w.shape
    s = s0.astype(np.float64).copy()
    y = np.zeros((T, C))
    for t in range(T):
        for hd in range(H):
            sl = slice(hd * S, (hd + 1) * S)
            a = np.outer(k[t, sl], v[t, sl])
            y[t, sl] = r[t, sl] @ (u[hd][:, None] * a + s[hd])
            s[hd] = w[hd][:, None] * s[hd] + a
    return y, s


def test_wkv5_scan_matches_brute_force_and_explicit_sum():
    T, H, S = 9, 3, 64
    C = H * S
    r, k, v = (rng.standard_normal((T, C)).astype(np.float32) for _ in range(3))
    w = np.exp(-np.exp(rng.uniform(-6, 0, (H, S)))).astype(np.float32)
    u = rng.uniform(-1, 1, (H, S)).astype(np.float32)
    s0 = rng.standard_normal((H, S, S)).astype(np.float32)
    y, s = po.wkv5_2_seq_f32(s0, r, k, v, w, u)
    yb, sb = _wkv5_brute(*(a.astype(np.float64) for a in (r, k, v, w, u)), s0)
    assert np.allclose(y, yb, rtol=1e-4, atol=1e-4)
    assert np.allclose(s, sb, rtol=1e-4, atol=1e-4)
    # S_T = diag(w)^T S_0 + sum_i diag(w)^(T-1-i) k_i v_i^T
    for hd in range(H):
        sl = slice(hd * S, (hd + 1) * S)
        ex = (w[hd].astype(np.float64) ** T)[:, None] * s0[hd]
        for i in range(T):
            ex += (w[hd].astype(np.float64) ** (T - 1 - i))[:, None] * np.outer(k[i, sl], v[i, sl])
        assert np.allclose(s[hd], ex, rtol=1e-4, atol=1e-4)


def test_wkv5_0_matrix_form_matches_brute_force_scan():
    """RWKV-5.0 (att_seq.cu:181-243): the matrix form with decay powers must equal the
    recurrence with one decay / bonus per head, outputs and final state."""
    T, H, S = 11, 3, 64
    C = H * S
    r, k, v = (rng.standard_normal((T, C)).astype(np.float32) for _ in range(3))
    w = np.exp(-np.exp(rng.uniform(-6, 0, H))).astype(np.float32)
    u = rng.uniform(-1, 1, H).astype(np.float32)
    s0 = rng.standard_normal((H, S, S)).astype(np.float32)
    y, s = po.wkv5_seq_matrix_f32(s0, r, k, v, w, u)
    wb = np.repeat(w[:, None], S, axis=1).astype(np.float64)
    ub = np.repeat(u[:, None], S, axis=1).astype(np.float64)
    yb, sb = _wkv5_brute(*(a.astype(np.float64) for a in (r, k, v)), wb, ub, s0)
    assert np.allclose(y, yb, rtol=2e-4, atol=2e-4)
    assert np.allclose(s, sb, rtol=2e-4, atol=2e-4)
    # T = 1: out = r.(u k v^T + S), S' = w S + k v^T exactly as the one-token functor (att.cu:64-81)
    y1, s1 = po.wkv5_seq_matrix_f32(s0, r[:1], k[:1], v[:1], w, u)
    for hd in range(H):
        sl = slice(hd * S, (hd + 1) * S)
        a = np.outer(k[0, sl], v[0, sl]).astype(np.float64)
        assert np.allclose(y1[0, sl], r[0, sl].astype(np.float64) @ (u[hd] * a + s0[hd]), rtol=1e-4, atol=1e-4)
        assert np.allclose(s1[hd], w[hd] * s0[hd].astype(np.float64) + a, rtol=1e-5, atol=1e-5)


def test_att_v5_0_seq_equals_loop_of_one_token_steps():
    """The cross-formulation invariant of RWKV-5.0: att_seq_v5 (matrix form) over T rows equals
    T calls of att_one_v5 (functor form) carrying the state (model_forward_seq.cpp:34-46)."""
    T, H, S = 7, 2, 64
    C = H * S
    h = np.float16
    x = rng.standard_normal((T, C)).astype(h)
    sx = rng.standard_normal(C).astype(h)
    s0 = (0.1 * rng.standard_normal((H, S, S))).astype(np.float32)
    ln_w, ln_b = (1 + 0.05 * rng.standard_normal(C)).astype(h), (0.05 * rng.standard_normal(C)).astype(h)
    lx_w, lx_b = (1 + 0.05 * rng.standard_normal(C)).astype(np.float32), (0.05 * rng.standard_normal(C)).astype(np.float32)
    mk, mv, mr = (rng.uniform(0, 1, C).astype(h) for _ in range(3))
    td = np.exp(-np.exp(rng.uniform(-6, 0, H))).astype(np.float32)
    tf = rng.uniform(-1, 1, H).astype(np.float32)
    kw, vw, rw, ow = ((0.05 * rng.standard_normal((C, C))).astype(h) for _ in range(4))
    ys, xxs, ss = po.att_v5_0_f16(x, sx, s0, ln_w, ln_b, lx_w, lx_b, mk, mv, mr, td, tf, kw, vw, rw, ow, H)
    s, shift = s0, sx
    for t in range(T):
        y1, shift, s = po.att_v5_0_f16(x[t], shift, s, ln_w, ln_b, lx_w, lx_b, mk, mv, mr, td, tf, kw, vw, rw, ow, H)
        d = np.abs(y1.astype(np.float32) - ys[t].astype(np.float32)).max()
        assert d <= 4e-3, (t, d)
    assert np.array_equal(shift, xxs)
    assert np.allclose(s, ss, rtol=1e-4, atol=1e-4)
    # without a gate and with w, u constant over a head, the 5.1 functor path gives the same token
    y51, _, s51 = po.att_v5_2_f16(x[0], sx, s0, ln_w, ln_b, lx_w, lx_b, mk, mv, mr, mr,
                                  np.repeat(td[:, None], S, 1), np.repeat(tf[:, None], S, 1), kw, vw, rw,
                                  np.zeros((C, C), h), ow, H)
    _, _, s50 = po.att_v5_0_f16(x[0], sx, s0, ln_w, ln_b, lx_w, lx_b, mk, mv, mr, td, tf, kw, vw, rw, ow, H)
    assert np.array_equal(s51, s50)  # same state update; the outputs differ by the gate


# ---------------------------------------------------------------- dequant u8
def _dequant_numpy(q, mx, rx, my, ry):
    """Independent numpy statement of the dequantisation: c = rx/255, a = c*ry, b = mx+my in
    float32 (numpy's float32 operations are correctly rounded), the fused multiply-add exactly
    in the 64-bit-mantissa long double (q*a has <= 32 significant bits; the widest exponent gap
    to b on the grid below is 2^27), then one rounding to float32 and one to float16."""
    assert np.finfo(np.longdouble).nmant >= 63
    f = np.float32
    c = rx.astype(f) / f(255)
    a = c[None, :] * ry.astype(f)[:, None]
    b = mx.astype(f)[None, :] + my.astype(f)[:, None]
    exact = q.astype(np.longdouble) * a.astype(np.longdouble) + b.astype(np.longdouble)
    return exact.astype(f).astype(np.float16)


def test_dequant_all_codes_times_scale_grid_bit_exact():
    q = np.arange(256, dtype=np.uint8)[:, None].repeat(64, axis=1)  # K=256 rows: code = row index
    mxs = h([-0.09, -0.031, 0.0, 0.0123, -1.7, 3e-5, -0.5, 2.0])
    rxs = h([0.17, 0.011, 1.0, 0.33, 5.5, 1e-3, 0.0625, 2.5e-4])
    N = 64
    mx = np.tile(mxs, 8)
    rx = np.repeat(rxs, 8)
    for my_v, ry_v in [(-0.07, 0.93), (0.0, 1.0), (0.011, 0.5), (-2.0, 0.031), (6e-5, 0.999)]:
        my = np.full(256, my_v, np.float16)
        ry = np.full(256, ry_v, np.float16)
        got = po.dequant_u8(q, mx, rx, my, ry)
        ref = _dequant_numpy(q, mx, rx, my, ry)
        assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))
    # scalar entry point agrees with the matrix one
    s = po.lib.orc_dequant_u8_scalar(200, int(mx[3].view(np.uint16)), int(rx[3].view(np.uint16)),
                                     int(my[0].view(np.uint16)), int(ry[0].view(np.uint16)))
    assert s == got[200, 3].view(np.uint16)
    assert N == got.shape[1]


def test_quantise_then_dequantise_error_is_half_a_step():
    K, N = 192, 160
    w = h(rng.standard_normal((K, N)) * 0.02)
    q, mx, rx, my, ry = quantize_u8(w)
    assert q.min() == 0 and q.max() == 255
    wd = po.dequant_u8(q, mx, rx, my, ry).astype(np.float64)
    step = rx.astype(np.float64)[None, :] * ry.astype(np.float64)[:, None] / 255
    err = np.abs(wd - w.astype(np.float64))
    assert (err <= 0.5 * step + 3e-4).all()  # half a step + binary16 rounding of a,b,w^
    assert err.mean() < 0.3 * step.mean() + 1e-4


# ---------------------------------------------------------------- one-token product on uint8 codes
def _weights_f32_numpy(q, mx, rx, my, ry):
    """The fp32 weight of every code by the dequantisation formula, before any rounding to half
    (same independent statement as _dequant_numpy, stopped one rounding earlier)."""
    f = np.float32
    c = rx.astype(f) / f(255)
    a = c[None, :] * ry.astype(f)[:, None]
    b = mx.astype(f)[None, :] + my.astype(f)[:, None]
    return (q.astype(np.longdouble) * a.astype(np.longdouble) + b.astype(np.longdouble)).astype(f)


def test_gemv_u8_one_hot_rows_return_the_unrounded_fp32_weights():
    K, N = 96, 130
    w = h(rng.standard_normal((K, N)) * 0.02)
    q, mx, rx, my, ry = quantize_u8(w)
    want = _weights_f32_numpy(q, mx, rx, my, ry)
    assert (want.astype(np.float16).astype(np.float32) != want).mean() > 0.9  # i.e. not the binary16 w^
    for k in (0, 1, 37, K - 1):
        e = np.zeros(K, np.float16)
        e[k] = 1
        assert np.array_equal(po.gemv_u8(e, q, mx, rx, my, ry), want[k]), k  # catches a transposed q, swapped mx/my
        e[k] = -2
        assert np.array_equal(po.gemv_u8(e, q, mx, rx, my, ry), -2 * want[k]), k


def test_gemv_u8_against_float64_of_the_real_valued_formula():
    for K, N in ((512, 200), (2048, 65), (16, 1)):
        w = h(rng.standard_normal((K, N)) * 0.02)
        q, mx, rx, my, ry = quantize_u8(w)
        x = h(rng.standard_normal(K) * 3)
        f = np.float64
        real = q.astype(f) * (rx.astype(f) / 255)[None, :] * ry.astype(f)[:, None] + mx.astype(f)[None, :] + my.astype(f)[:, None]
        exact = x.astype(f) @ real
        mag = np.abs(x.astype(f)) @ np.abs(real)
        got = po.gemv_u8(x, q, mx, rx, my, ry)
        # every fp32 weight is within 1.5 fp32 roundings of the real value; the sum is rounded once
        assert (np.abs(got - exact) <= 2.0 ** -22 * mag + 1e-30).all()
        # and it is the exact sum of x times the fp32 weights
        w32 = _weights_f32_numpy(q, mx, rx, my, ry)
        assert np.array_equal(got, (x.astype(f) @ w32.astype(f)).astype(np.float32))


def test_registered_codes_change_one_token_products_only():
    K, N = 256, 96
    w = h(rng.standard_normal((K, N)) * 0.02)
    q, mx, rx, my, ry = quantize_u8(w)
    W = po.dequant_u8(q, mx, rx, my, ry)
    x2 = h(rng.standard_normal((2, K)))
    before1, before2 = po.gemm_f16(x2[0], W, "f32"), po.gemm_f16(x2, W, "f32")
    po.register_u8(W, q, mx, rx, my, ry)
    try:
        assert np.array_equal(po.gemm_f16(x2[0], W, "f32"), po.gemv_u8(x2[0], q, mx, rx, my, ry))
        assert not np.array_equal(po.gemm_f16(x2[0], W, "f32"), before1)
        assert np.array_equal(po.gemm_f16(x2, W, "f32"), before2)   # matrix x matrix: the binary16 w^
        assert np.array_equal(po.gemm_f16(x2[0], W.copy(), "f32"), before1)  # keyed by the matrix, not by its values
    finally:
        po.unregister_u8(W)
    assert np.array_equal(po.gemm_f16(x2[0], W, "f32"), before1)
