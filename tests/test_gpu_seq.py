"""GPU parity tests of the seq-mode (prompt) operators against the oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import pyoracle as po
from hipref import DevBuf, L, assert_close_f16, dev, fr, make_weight

_alive = []


def keep(a):
    b = dev(a)
    _alive.append(b)
    if len(_alive) > 96:
        fr.check(L().frhip_device_sync())
        del _alive[:48]
    return b


rng = np.random.default_rng(777)


@pytest.fixture(autouse=True)
def _rng_per_test(request):
    """Every test draws from a generator seeded by its own name, so its data do not depend on which
    other tests ran before it (or on cases added to them)."""
    import zlib
    global rng
    rng = np.random.default_rng([777, zlib.crc32(request.node.name.encode())])


def h(x):
    return np.asarray(x, np.float32).astype(np.float16)


@pytest.mark.parametrize("T,K,N", [(1024, 2048, 2048), (512, 2560, 8960), (100, 8192, 2048), (1, 64, 128), (130, 128, 200), (7, 1792, 512),
                                   # wide enough for the variable-width tiles: ragged N (last block partial), ragged T
                                   (1024, 256, 7000), (900, 128, 6144),
                                   # one round of 256-row tiles beats two of 128-row tiles: the eight-wave form, full and ragged
                                   (1024, 128, 10240), (1000, 128, 10000)])
@pytest.mark.parametrize("quant", [False, True])
def test_gemm_against_oracle(T, K, N, quant):
    x = h(rng.standard_normal((T, K)))
    w = h(rng.standard_normal((K, N)) * 0.02)
    pw, wref = make_weight(w, quant)
    ref = po.gemm_f16(x, wref, "f32")
    y32, y16 = DevBuf.empty((T, N), np.float32), DevBuf.empty((T, N), np.float16)
    fr.check(L().frhip_gemm(keep(x).ptr, pw.ref, y32.ptr, T, fr.F32, None))
    fr.check(L().frhip_gemm(keep(x).ptr, pw.ref, y16.ptr, T, fr.F16, None))
    got = y32.numpy()
    tol = 3e-6 * np.sqrt(K) * np.abs(ref).max() + 1e-5
    assert np.abs(got - ref).max() <= tol, np.abs(got - ref).max()
    assert_close_f16(y16.numpy(), ref.astype(np.float16), max_ulp=1, what="gemm f16 out")
    # an asymmetric probe: row t = e_k picks out row k of the weight exactly (catches a swapped
    # operand or a wrong fragment layout that a random comparison could only show as noise)
    if T >= 4:
        e = np.zeros((T, K), np.float16)
        ks = [0, 1, K // 2 + 3, K - 1]
        for t, k in enumerate(ks):
            e[t, k] = 1
        fr.check(L().frhip_gemm(keep(e).ptr, pw.ref, y32.ptr, T, fr.F32, None))
        out = y32.numpy()
        for t, k in enumerate(ks):
            assert np.array_equal(out[t], wref[k].astype(np.float32)), (t, k)
        assert not out[len(ks):].any()


def test_gemm_sigmoid_and_silu_epilogues_every_binary16_bit_exact():
    """Every finite binary16 value goes through the product's sigmoid epilogue (identity weight, so the
    accumulator is the input exactly) and must come out as the oracle's double-evaluated sigmoid (and its silu), bit for bit;
    once on 64-row tiles (T = 1024, N = 64) and once on the variable-width tiles (N = 8192, columns repeat)."""
    bits = np.arange(65536, dtype=np.uint16)
    x = bits.view(np.float16).copy()
    x[~np.isfinite(x)] = 0
    x[bits == 0x8000] = 0  # the accumulator of 0 + (-0)(1) is +0: -0 cannot reach the epilogue this way
    a = x.reshape(1024, 64)
    want = po.sigmoid_f16(a)
    want_silu = po.silu_f16(a)
    for N in (64, 8192):
        w = np.zeros((64, N), np.float16)
        w[np.arange(N) % 64, np.arange(N)] = 1
        pw = fr.PackedWeight(w_kn=w)
        y = DevBuf.empty((1024, N), np.float16)
        for act, ref in ((2, want), (4, want_silu)):  # FRHIP_ACT_SIGMOID, FRHIP_ACT_SILU
            fr.check(L().frhip_gemm_act(keep(a).ptr, pw.ref, y.ptr, 1024, act, None))
            got = y.numpy()
            for c0 in range(0, N, 64):
                assert np.array_equal(got[:, c0:c0 + 64].view(np.uint16), ref.view(np.uint16)), (act, c0)


def test_gemm_act_relu2_and_silu_match_the_oracle():
    x = h(rng.standard_normal((256, 128)))
    w = h(rng.standard_normal((128, 192)) * 0.1)
    pw = fr.PackedWeight(w_kn=w)
    lin = po.gemm_f16(x, w, "f16")
    y = DevBuf.empty((256, 192), np.float16)
    fr.check(L().frhip_gemm_act(keep(x).ptr, pw.ref, y.ptr, 256, 3, None))
    t = lin.astype(np.float16)
    assert_close_f16(y.numpy(), np.where(t > 0, t * t, np.float16(0)).astype(np.float16), max_ulp=4, max_frac=0.05, what="relu2")  # one spacing of t is two of t*t
    assert L().frhip_gemm_act(keep(x).ptr, pw.ref, y.ptr, 256, 7, None) == -1


def test_gemm_rejects_bad_shapes():
    w = fr.PackedWeight(w_kn=h(rng.standard_normal((96, 64))))
    y = DevBuf.empty((4, 64), np.float32)
    assert L().frhip_gemm(keep(h(np.zeros((4, 96)))).ptr, w.ref, y.ptr, 4, fr.F32, None) == -2  # K % 64
    assert L().frhip_gemm(None, w.ref, y.ptr, 4, fr.F32, None) == -1


def _common(C_):
    return (h(1 + 0.1 * rng.standard_normal(C_)), h(0.1 * rng.standard_normal(C_)))


# (1024, 2048, 8192): r and k as separate one-round launches, the value product split over K in two slices;
# (300, 2048, 8192): the value product in four slices over ragged row tiles; (512, 2560, 8960): three slices of 47, 47 and 46 K-steps
# (16, 2048, 8192), (130, 2048, 8192), (200, 2560, 8960): short prompts at full width -- products split over K across the idle compute
# units: r,k grouped in one split launch (16 rows), product by product because the group is too wide (130, 200 rows), the value
# product in 16 and in fewer slices
@pytest.mark.parametrize("T,C_,F_", [(64, 512, 1792), (300, 2048, 8192), (1024, 2048, 8192), (512, 2560, 8960), (1, 512, 1024), (33, 768, 3072), (3000, 512, 1792),
                                     (16, 2048, 8192), (130, 2048, 8192), (200, 2560, 8960)])
@pytest.mark.parametrize("quant", [False, True])
def test_ffn_seq(T, C_, F_, quant):
    g = np.random.default_rng(5000 + T) if T >= 512 else rng  # the full-size cases draw from a stream of their own
    x, sx = h(g.standard_normal((T, C_)) * 2), h(g.standard_normal(C_))
    ln_w, ln_b = h(1 + 0.1 * g.standard_normal(C_)), h(0.1 * g.standard_normal(C_))
    mk, mr = h(g.uniform(0, 1, C_)), h(g.uniform(0, 1, C_))
    kw, kref = make_weight(h(g.standard_normal((C_, F_)) * 0.02), quant)
    vw, vref = make_weight(h(g.standard_normal((F_, C_)) * 0.02), quant)
    rw, rref = make_weight(h(g.standard_normal((C_, C_)) * 0.02), quant)
    ref_x, ref_xx = po.ffn_f16(x, sx, ln_w, ln_b, mk, mr, kref, vref, rref)
    x_out, xx_out = DevBuf.empty((T, C_), np.float16), DevBuf.empty(C_, np.float16)
    ws = DevBuf(L().frhip_seq_workspace_bytes(T, C_, F_))
    fr.check(L().frhip_ffn_seq(T, C_, F_, keep(x).ptr, keep(sx).ptr, keep(ln_w).ptr, keep(ln_b).ptr, keep(mk).ptr,
                               keep(mr).ptr, kw.ref, vw.ref, rw.ref, x_out.ptr, xx_out.ptr, 0, ws.ptr, None))
    assert_close_f16(xx_out.numpy(), ref_xx, max_ulp=1, what="xx_last")
    assert_close_f16(x_out.numpy(), ref_x, max_ulp=3, max_frac=0.2, what="x_out", floor_rms=1.0)


@pytest.mark.parametrize("T,C_,F_", [(64, 512, 1792), (1024, 2048, 8192), (1, 512, 1024), (200, 768, 3072)])
@pytest.mark.parametrize("quant", [False, True])
def test_ffn_seq_with_the_halving_folded_in(T, C_, F_, quant):
    """post_div2 = 1: the rows leave halved in binary16 after the residual, the bits of scalar_div_(x_out, 2) on
    the result without it (model_forward_seq.cpp:163-165 halves the rows after every sixth layer); in the
    launch split over K the halving sits in the reduction pass."""
    g = np.random.default_rng(7000 + T)
    x, sx = h(g.standard_normal((T, C_)) * 2), h(g.standard_normal(C_))
    ln_w, ln_b = h(1 + 0.1 * g.standard_normal(C_)), h(0.1 * g.standard_normal(C_))
    mk, mr = h(g.uniform(0, 1, C_)), h(g.uniform(0, 1, C_))
    kw, _ = make_weight(h(g.standard_normal((C_, F_)) * 0.02), quant)
    vw, _ = make_weight(h(g.standard_normal((F_, C_)) * 0.02), quant)
    rw, _ = make_weight(h(g.standard_normal((C_, C_)) * 0.02), quant)
    ws = DevBuf(L().frhip_seq_workspace_bytes(T, C_, F_))
    outs = []
    for div2 in (0, 1):
        x_out, xx_out = DevBuf.empty((T, C_), np.float16), DevBuf.empty(C_, np.float16)
        fr.check(L().frhip_ffn_seq(T, C_, F_, keep(x).ptr, keep(sx).ptr, keep(ln_w).ptr, keep(ln_b).ptr, keep(mk).ptr,
                                   keep(mr).ptr, kw.ref, vw.ref, rw.ref, x_out.ptr, xx_out.ptr, div2, ws.ptr, None))
        outs.append((x_out.numpy(), xx_out.numpy()))
    assert np.array_equal(outs[1][0], outs[0][0] / np.float16(2))
    assert np.array_equal(outs[1][1], outs[0][1])  # the shift state is LN(x) of the last row: not halved


def _state_v4(C_, fresh):
    if fresh:
        return np.zeros(C_, np.float32), np.zeros(C_, np.float32), np.full(C_, -1e30, np.float32)
    return (rng.standard_normal(C_).astype(np.float32), rng.uniform(0.5, 3, C_).astype(np.float32),
            rng.standard_normal(C_).astype(np.float32))


@pytest.mark.parametrize("T,C_", [(64, 512), (1024, 2048), (1, 512), (37, 768), (3000, 512), (24, 2048), (150, 2048)])  # 3000: a long, ragged prompt (94 chunks); 24, 150: short prompts at full width (split products)
@pytest.mark.parametrize("quant", [False, True])
@pytest.mark.parametrize("fresh", [True, False])
def test_att_seq_v4(T, C_, quant, fresh):
    x, sx = h(rng.standard_normal((T, C_)) * 2), h(rng.standard_normal(C_))
    aa, bb, pp = _state_v4(C_, fresh)
    ln_w, ln_b = _common(C_)
    mixes = [h(rng.uniform(0, 1, C_)) for _ in range(3)]
    td = (-np.exp(rng.uniform(-5, 1, C_))).astype(np.float32)
    tf = rng.uniform(-1, 1, C_).astype(np.float32)
    ws_, refs = [], []
    for _ in range(4):
        w, r = make_weight(h(rng.standard_normal((C_, C_)) * 0.02), quant)
        ws_.append(w)
        refs.append(r)
    ref = po.att_seq_v4_f16(x, sx, aa, bb, pp, ln_w, ln_b, *mixes, td, tf, *refs)
    x_out, xx_out = DevBuf.empty((T, C_), np.float16), DevBuf.empty(C_, np.float16)
    ao, bo, po_ = (DevBuf.empty(C_, np.float32) for _ in range(3))
    ws = DevBuf(L().frhip_seq_workspace_bytes(T, C_, 4 * C_))
    fr.check(L().frhip_att_seq_v4(T, C_, keep(x).ptr, keep(sx).ptr, keep(aa).ptr, keep(bb).ptr, keep(pp).ptr,
                                  keep(ln_w).ptr, keep(ln_b).ptr, *[keep(m).ptr for m in mixes], keep(td).ptr,
                                  keep(tf).ptr, *[w.ref for w in ws_], x_out.ptr, xx_out.ptr, ao.ptr, bo.ptr, po_.ptr,
                                  ws.ptr, None))
    assert_close_f16(xx_out.numpy(), ref[1], max_ulp=1, what="xx_last")
    assert_close_f16(x_out.numpy(), ref[0], max_ulp=3, max_frac=0.1, what="x_out")
    # the carried state: same value, possibly another exponent offset pp -> compare aa*e^pp etc.
    for got, want in ((ao, ref[2]), (bo, ref[3])):
        g = got.numpy().astype(np.float64) * np.exp(po_.numpy().astype(np.float64) - ref[4].astype(np.float64))
        assert np.allclose(g, want, rtol=2e-3, atol=2e-3 * np.abs(want).max())
    assert np.abs(po_.numpy() - ref[4]).max() < 30  # offsets stay in a sane range


@pytest.mark.parametrize("T,C_", [(1024, 2048), (700, 512), (5000, 256)])  # 5000: beyond 128 chunks of 32 steps, the scan's serial pass
def test_att_seq_v4_state_updated_in_place_equals_separate_outputs(T, C_):
    """The header allows aa_out / bb_out / pp_out to be the buffers of aa / bb / pp (as frhip_att_one_v4 does).
    The scan's last chunk writes them while other chunks may not have started: every pass must take the
    incoming state from the copy the first pass makes.  Bit for bit the same as with separate outputs."""
    x, sx = h(rng.standard_normal((T, C_)) * 2), h(rng.standard_normal(C_))
    aa, bb, pp = _state_v4(C_, False)
    ln_w, ln_b = _common(C_)
    mixes = [h(rng.uniform(0, 1, C_)) for _ in range(3)]
    td = (-np.exp(rng.uniform(-5, 1, C_))).astype(np.float32)
    tf = rng.uniform(-1, 1, C_).astype(np.float32)
    pairs = [make_weight(h(rng.standard_normal((C_, C_)) * 0.02), False) for _ in range(4)]
    ws_, refs = [p[0] for p in pairs], [p[1] for p in pairs]
    ws = DevBuf(L().frhip_seq_workspace_bytes(T, C_, 4 * C_))
    dx, dsx = keep(x), keep(sx)
    consts = [keep(a).ptr for a in (ln_w, ln_b, *mixes, td, tf)]
    results = []
    for in_place in (False, True):
        st = [dev(aa), dev(bb), dev(pp)]
        outs = st if in_place else [DevBuf.empty(C_, np.float32) for _ in range(3)]
        x_out, xx_out = DevBuf.empty((T, C_), np.float16), DevBuf.empty(C_, np.float16)
        fr.check(L().frhip_att_seq_v4(T, C_, dx.ptr, dsx.ptr, st[0].ptr, st[1].ptr, st[2].ptr, *consts,
                                      *[w.ref for w in ws_], x_out.ptr, xx_out.ptr, outs[0].ptr, outs[1].ptr, outs[2].ptr,
                                      ws.ptr, None))
        results.append([x_out.numpy(), xx_out.numpy()] + [o.numpy() for o in outs])
    for sep, inp in zip(*results):
        assert np.array_equal(sep, inp)
    if T == 5000:  # the long prompt against the oracle as well (the serial pass is otherwise only reached by a switch)
        ref = po.att_seq_v4_f16(x, sx, aa, bb, pp, ln_w, ln_b, *mixes, td, tf, *refs)
        assert_close_f16(results[0][0], ref[0], max_ulp=3, max_frac=0.1, what="x_out, T = 5000")


@pytest.mark.parametrize("T,C_,H_", [(48, 512, 8), (512, 2560, 40), (1, 512, 8), (77, 512, 8), (3000, 512, 8), (40, 2560, 40)])  # (40, 2560, 40): k,v,r,g of a short prompt in one split launch
@pytest.mark.parametrize("quant", [False, True])
def test_att_seq_v5_2(T, C_, H_, quant):
    S_ = C_ // H_
    x, sx = h(rng.standard_normal((T, C_)) * 2), h(rng.standard_normal(C_))
    s = rng.standard_normal((H_, S_, S_)).astype(np.float32)
    ln_w, ln_b = _common(C_)
    lx_w = (1 + 0.1 * rng.standard_normal(C_)).astype(np.float32)
    lx_b = (0.1 * rng.standard_normal(C_)).astype(np.float32)
    mixes = [h(rng.uniform(0, 1, C_)) for _ in range(4)]
    td = np.exp(-np.exp(rng.uniform(-6, 0, (H_, S_)))).astype(np.float32)
    tf = rng.uniform(-1, 1, (H_, S_)).astype(np.float32)
    ws_, refs = [], []
    for _ in range(5):
        w, r = make_weight(h(rng.standard_normal((C_, C_)) * 0.02), quant)
        ws_.append(w)
        refs.append(r)
    ref_x, ref_xx, ref_s = po.att_v5_2_f16(x if T > 1 else x[0], sx, s, ln_w, ln_b, lx_w, lx_b, *mixes, td, tf, *refs, H_)
    x_out, xx_out = DevBuf.empty((T, C_), np.float16), DevBuf.empty(C_, np.float16)
    s_out = DevBuf.empty((H_, S_, S_), np.float32)
    ws = DevBuf(L().frhip_seq_workspace_bytes(T, C_, 4 * C_))
    fr.check(L().frhip_att_seq_v5_2(T, C_, H_, keep(x).ptr, keep(sx).ptr, keep(s).ptr, keep(ln_w).ptr, keep(ln_b).ptr,
                                    keep(lx_w).ptr, keep(lx_b).ptr, *[keep(m).ptr for m in mixes], keep(td).ptr,
                                    keep(tf).ptr, *[w.ref for w in ws_], x_out.ptr, xx_out.ptr, s_out.ptr, ws.ptr,
                                    None))
    assert_close_f16(xx_out.numpy(), ref_xx, max_ulp=1, what="xx_last")
    assert np.allclose(s_out.numpy(), ref_s, rtol=1e-4, atol=1e-4 * np.abs(ref_s).max())
    assert_close_f16(x_out.numpy().reshape(ref_x.shape), ref_x, max_ulp=4, max_frac=0.2, what="x_out", floor_rms=1.0)


@pytest.mark.parametrize("T,C_,H_", [(48, 512, 8), (300, 2048, 32), (1, 512, 8), (77, 512, 8)])
@pytest.mark.parametrize("quant", [False, True])
def test_att_seq_v5(T, C_, H_, quant):
    """RWKV-5.0 seq attention against the oracle's matrix form (kernels/cuda/att_seq.cu:158-256)."""
    S_ = C_ // H_
    x, sx = h(rng.standard_normal((T, C_)) * 2), h(rng.standard_normal(C_))
    s = rng.standard_normal((H_, S_, S_)).astype(np.float32)
    ln_w, ln_b = _common(C_)
    lx_w = (1 + 0.1 * rng.standard_normal(C_)).astype(np.float32)
    lx_b = (0.1 * rng.standard_normal(C_)).astype(np.float32)
    mixes = [h(rng.uniform(0, 1, C_)) for _ in range(3)]
    td = np.exp(-np.exp(rng.uniform(-6, 0, H_))).astype(np.float32)
    tf = rng.uniform(-1, 1, H_).astype(np.float32)
    ws_, refs = [], []
    for _ in range(4):
        w, r = make_weight(h(rng.standard_normal((C_, C_)) * 0.02), quant)
        ws_.append(w)
        refs.append(r)
    ref_x, ref_xx, ref_s = po.att_v5_0_f16(x if T > 1 else x[0], sx, s, ln_w, ln_b, lx_w, lx_b, *mixes, td, tf, *refs, H_)
    x_out, xx_out = DevBuf.empty((T, C_), np.float16), DevBuf.empty(C_, np.float16)
    s_out = DevBuf.empty((H_, S_, S_), np.float32)
    ws = DevBuf(L().frhip_seq_workspace_bytes(T, C_, 4 * C_))
    fr.check(L().frhip_att_seq_v5(T, C_, H_, keep(x).ptr, keep(sx).ptr, keep(s).ptr, keep(ln_w).ptr, keep(ln_b).ptr,
                                  keep(lx_w).ptr, keep(lx_b).ptr, *[keep(m).ptr for m in mixes], keep(td).ptr,
                                  keep(tf).ptr, *[w.ref for w in ws_], x_out.ptr, xx_out.ptr, s_out.ptr, ws.ptr,
                                  None))
    assert_close_f16(xx_out.numpy(), ref_xx, max_ulp=1, what="xx_last")
    assert np.allclose(s_out.numpy(), ref_s, rtol=1e-4, atol=1e-4 * np.abs(ref_s).max())
    assert_close_f16(x_out.numpy().reshape(ref_x.shape), ref_x, max_ulp=4, max_frac=0.2, what="x_out", floor_rms=1.0)
