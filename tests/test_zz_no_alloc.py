"""GPU test of the entry point that allocates nothing: frhip_ffn_one_static keeps its intermediate
vectors in a device array built into the library and must give frhip_ffn_one's result bit for bit."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from hipref import DevBuf, L, dev, fr, make_weight


def h(x):
    return np.asarray(x, np.float32).astype(np.float16)


def _case(C_, F_, quant, seed, div2):
    g = np.random.default_rng(seed)
    x, sx = h(g.standard_normal(C_) * 2), h(g.standard_normal(C_))
    ln_w, ln_b = h(1 + 0.1 * g.standard_normal(C_)), h(0.1 * g.standard_normal(C_))
    mk, mr = h(g.uniform(0, 1, C_)), h(g.uniform(0, 1, C_))
    kw, _ = make_weight(h(g.standard_normal((C_, F_)) * 0.02), quant)
    vw, _ = make_weight(h(g.standard_normal((F_, C_)) * 0.02), quant)
    rw, _ = make_weight(h(g.standard_normal((C_, C_)) * 0.02), quant)
    bufs = [dev(a) for a in (x, sx, ln_w, ln_b, mk, mr)]
    ws = DevBuf(L().frhip_decode_workspace_bytes(C_, F_))
    want_x, want_xx = DevBuf.empty(C_, np.float16), DevBuf.empty(C_, np.float16)
    got_x, got_xx = DevBuf.empty(C_, np.float16), DevBuf.empty(C_, np.float16)
    fr.check(L().frhip_ffn_one(C_, F_, *[b.ptr for b in bufs], kw.ref, vw.ref, rw.ref, want_x.ptr, want_xx.ptr, div2,
                               ws.ptr, None), "ffn_one")
    fr.check(L().frhip_ffn_one_static(C_, F_, *[b.ptr for b in bufs], kw.ref, vw.ref, rw.ref, got_x.ptr, got_xx.ptr,
                                      div2, None), "ffn_one_static")
    fr.check(L().frhip_device_sync())
    wx, gx = want_x.numpy(), got_x.numpy()
    assert np.isfinite(wx.astype(np.float32)).all() and np.abs(wx.astype(np.float32)).max() > 0
    assert np.array_equal(gx.view(np.uint16), wx.view(np.uint16)), "x_out differs from frhip_ffn_one"
    assert np.array_equal(got_xx.numpy().view(np.uint16), want_xx.numpy().view(np.uint16)), "xx_out differs"


@pytest.mark.parametrize("quant", [False, True])
def test_static_scratch_entry_point_equals_the_workspace_one_on_two_calls_in_a_row(quant):
    """Two calls in a row through the C ABI, the second with a smaller input: the array keeps the first
    call's contents, and nothing of them may show in the second result."""
    _case(2048, 8192, quant, seed=11, div2=0)
    _case(512, 1792, quant, seed=12, div2=1)


def test_static_scratch_entry_point_rejects_sizes_beyond_its_array():
    g = np.random.default_rng(3)
    C_, F_ = 256, 16384 + 256
    kw, _ = make_weight(h(g.standard_normal((C_, F_)) * 0.02))
    vw, _ = make_weight(h(g.standard_normal((F_, C_)) * 0.02))
    rw, _ = make_weight(h(g.standard_normal((C_, C_)) * 0.02))
    v = [dev(h(np.zeros(C_))) for _ in range(8)]
    rc = L().frhip_ffn_one_static(C_, F_, *[b.ptr for b in v[:6]], kw.ref, vw.ref, rw.ref, v[6].ptr, v[7].ptr, 0, None)
    assert rc == -2 and b"16384" in L().frhip_error_string()
