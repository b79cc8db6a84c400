"""GPU parity tests of the fused one-token operators and of whole-model greedy decode."""
import ctypes as C
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import pyoracle as po
from hipref import DevBuf, HipModelV4, L, assert_close_f16, dev, fr, greedy_against_oracle, make_weight
from synth import make_model

_alive = []


def keep(a):
    """Upload and keep the buffer alive until the test module is torn down (a temporary
    DevBuf would be freed as soon as its .ptr has been read)."""
    b = dev(a)
    _alive.append(b)
    if len(_alive) > 64:
        fr.check(L().frhip_device_sync())
        del _alive[:32]
    return b


rng = np.random.default_rng(321)


@pytest.fixture(autouse=True)
def _rng_per_test(request):
    """Every test draws from a generator seeded by its own name, so its data do not depend on which
    other tests ran before it (or on cases added to them)."""
    import zlib
    global rng
    rng = np.random.default_rng([321, zlib.crc32(request.node.name.encode())])


def h(x):
    return np.asarray(x, np.float32).astype(np.float16)


def _att_inputs(C_):
    return dict(
        x=h(rng.standard_normal(C_) * 2), sx=h(rng.standard_normal(C_)),
        aa=rng.standard_normal(C_).astype(np.float32), bb=rng.uniform(0.5, 3, C_).astype(np.float32),
        pp=rng.standard_normal(C_).astype(np.float32),
        ln_w=h(1 + 0.1 * rng.standard_normal(C_)), ln_b=h(0.1 * rng.standard_normal(C_)),
        mk=h(rng.uniform(0, 1, C_)), mv=h(rng.uniform(0, 1, C_)), mr=h(rng.uniform(0, 1, C_)),
        td=(-np.exp(rng.uniform(-5, 1, C_))).astype(np.float32), tf=rng.uniform(-1, 1, C_).astype(np.float32))


@pytest.mark.parametrize("C_", [2048, 768, 512, 5120, 4112])  # 5120, 4112: wider than the fused kernel, separate launches (4112: ragged last groups)
@pytest.mark.parametrize("quant", [False, True])
@pytest.mark.parametrize("fresh_state", [False, True])
def test_att_one_v4(C_, quant, fresh_state):
    i = _att_inputs(C_)
    if fresh_state:  # model.cpp:152-160
        i["aa"], i["bb"], i["pp"] = np.zeros(C_, np.float32), np.zeros(C_, np.float32), np.full(C_, -1e30, np.float32)
    ws, refs = [], []
    for _ in range(4):
        w, r = make_weight(h(rng.standard_normal((C_, C_)) * 0.02), quant)
        ws.append(w)
        refs.append(r)
    # at the wider shape the oracle multiplies the unrounded uint8 weights too, as the kernels do: the
    # difference between the two evaluations grows with sqrt(K) and would need a looser bound
    coded = quant and C_ > 4096
    if coded:
        for w, r in zip(ws, refs):
            po.register_u8(r, *w.parts)
    try:
        ref = po.att_one_v4_f16(i["x"], i["sx"], i["aa"], i["bb"], i["pp"], i["ln_w"], i["ln_b"], i["mk"], i["mv"],
                                i["mr"], i["td"], i["tf"], *refs)
    finally:
        if coded:
            for r in refs:
                po.unregister_u8(r)
    d = {k: keep(v) for k, v in i.items()}
    x_out, xx_out = DevBuf.empty(C_, np.float16), DevBuf.empty(C_, np.float16)
    aa_o, bb_o, pp_o = (DevBuf.empty(C_, np.float32) for _ in range(3))
    wsb = DevBuf(L().frhip_decode_workspace_bytes(C_, 4 * C_))
    fr.check(L().frhip_att_one_v4(C_, d["x"].ptr, d["sx"].ptr, d["aa"].ptr, d["bb"].ptr, d["pp"].ptr, d["ln_w"].ptr,
                                  d["ln_b"].ptr, d["mk"].ptr, d["mv"].ptr, d["mr"].ptr, d["td"].ptr, d["tf"].ptr,
                                  ws[0].ref, ws[1].ref, ws[2].ref, ws[3].ref, x_out.ptr, xx_out.ptr,
                                  aa_o.ptr, bb_o.ptr, pp_o.ptr, wsb.ptr, None))
    assert_close_f16(xx_out.numpy(), ref[1], max_ulp=1, what="xx")
    # uint8: the kernels multiply by w^ before its rounding to binary16, the oracle after it:
    # more one-spacing flips, same bound on their size
    # (one layernorm output on the other side of a rounding boundary -- the statistics are summed in another order than
    # the oracle's -- shifts every product by a little and with it about a tenth of the outputs by one spacing)
    ln_flip = bool((xx_out.numpy() != ref[1]).any())
    assert_close_f16(x_out.numpy(), ref[0], max_ulp=2, max_frac=0.3 if (quant or ln_flip) else 0.03, what="x_out")
    for got, want, nm in ((aa_o, ref[2], "aa"), (bb_o, ref[3], "bb"), (pp_o, ref[4], "pp")):
        assert np.allclose(got.numpy(), want, rtol=2e-4, atol=(2e-3 * np.abs(want).max()) if (quant or ln_flip) else 2e-5), nm


# (2560, 10240), (4096, 16384): value rows longer than a register tiling (sliced kernel); (5120, 20480): also wider
# than the fused layernorm prologue
@pytest.mark.parametrize("C_,F_", [(2048, 8192), (768, 3072), (512, 1024), (2560, 10240), (4096, 16384), (5120, 20480)])
@pytest.mark.parametrize("quant", [False, True])
@pytest.mark.parametrize("div2", [0, 1])
def test_ffn_one(C_, F_, quant, div2):
    x, sx = h(rng.standard_normal(C_) * 2), h(rng.standard_normal(C_))
    ln_w, ln_b = h(1 + 0.1 * rng.standard_normal(C_)), h(0.1 * rng.standard_normal(C_))
    mk, mr = h(rng.uniform(0, 1, C_)), h(rng.uniform(0, 1, C_))
    kw, kref = make_weight(h(rng.standard_normal((C_, F_)) * 0.02), quant)
    vw, vref = make_weight(h(rng.standard_normal((F_, C_)) * 0.02), quant)
    rw, rref = make_weight(h(rng.standard_normal((C_, C_)) * 0.02), quant)
    if quant:  # the oracle's one-token products multiply the unrounded uint8 weights, as the kernels do
        for w, r in ((kw, kref), (vw, vref), (rw, rref)):
            po.register_u8(r, *w.parts)
    try:
        _ffn_one_checks(C_, F_, quant, div2, x, sx, ln_w, ln_b, mk, mr, kw, vw, rw, kref, vref, rref)
    finally:
        for r in (kref, vref, rref):
            po.unregister_u8(r)


def _ffn_one_checks(C_, F_, quant, div2, x, sx, ln_w, ln_b, mk, mr, kw, vw, rw, kref, vref, rref):
    ref_x, ref_xx = po.ffn_f16(x, sx, ln_w, ln_b, mk, mr, kref, vref, rref)
    if div2:
        ref_x = (ref_x.astype(np.float32) / 2).astype(np.float16)
    x_out, xx_out = DevBuf.empty(C_, np.float16), DevBuf.empty(C_, np.float16)
    wsb = DevBuf.empty(L().frhip_decode_workspace_bytes(C_, F_) // 2, np.float16)
    fr.check(L().frhip_ffn_one(C_, F_, keep(x).ptr, keep(sx).ptr, keep(ln_w).ptr, keep(ln_b).ptr, keep(mk).ptr, keep(mr).ptr,
                               kw.ref, vw.ref, rw.ref, x_out.ptr, xx_out.ptr, div2, wsb.ptr, None))
    assert_close_f16(xx_out.numpy(), ref_xx, max_ulp=1, what="xx")
    # A one-spacing flip in a few of the F relu^2 values moves many of the C outputs of
    # the last product by one spacing, so the end-to-end comparison is loose ...
    # (the number of flipped terms, and with it the bound, grows with the length of that product)
    loose = (4 if quant else 3) * max(1.0, (F_ / 8192) ** 0.5) + (2 if F_ > 8192 else 0)
    assert_close_f16(x_out.numpy(), ref_x, max_ulp=loose, max_frac=0.5 if quant else 0.3, what="x_out")
    # ... and the strict one restarts the oracle from the kernel's own intermediates
    # (workspace: binary16 rwkv | r | x_mid | g, fp32 k | v | r32, binary16 vx; each rounded up
    # to 256 bytes): bit-exact.
    ws = wsb.numpy()
    al = lambda n: (n + 255) // 256 * 256
    r_g = ws[al(2 * C_) // 2:][:C_]
    wide = 4 * al(2 * C_) if C_ > 4096 else 0  # the four mixed vectors of a wide model lie before vx
    vx_g = ws[(4 * al(2 * C_) + 3 * al(4 * C_) + wide) // 2:][:F_]
    xx_g = xx_out.numpy()  # the kernel's own layernorm output (checked against the oracle's above)
    r_ref = po.sigmoid_f16(po.gemm_f16(po.mix_f16(xx_g, sx, mr), rref, "f16"))
    vx_ref = po.relu_square_f16(po.gemm_f16(po.mix_f16(xx_g, sx, mk), kref, "f16"))
    # (where the receptance sum is negative, one spacing of it is several of the sigmoid's small output)
    assert_close_f16(r_g, r_ref, max_ulp=2, max_frac=0.1 if quant else 0.01, what="r")
    assert_close_f16(vx_g, vx_ref, max_ulp=6 if quant else 3, max_frac=0.3 if quant else 0.01, what="vx")  # a one-spacing flip of t becomes up to three in t*t
    if quant:
        # the last product against the real-valued weights, from the kernel's own r and vx
        out_e = (vx_g.astype(np.float64) @ vw.exact()).astype(np.float16)
        strict = np.array([po.lib.orc_hfma(int(a), int(b), int(c)) for a, b, c in
                           zip(out_e.view(np.uint16), r_g.view(np.uint16), x.view(np.uint16))], np.uint16).view(np.float16)
        if div2:
            strict = (strict.astype(np.float32) / 2).astype(np.float16)
        # The factored uint8 product sums F non-negative terms q * (vx * ry) in fp32 and subtracts almost all of
        # the sum again (mx * sum(vx)): its error grows with F (about 300 times the result at F = 16384), where
        # the result itself grows with sqrt(F).  Up to F = 8192 that stays within two spacings of the output.
        if F_ <= 8192:
            assert_close_f16(x_out.numpy(), strict, max_ulp=2, max_frac=0.02, what="x_out from kernel intermediates (uint8)")
            return
        # Beyond that, element by element: the kernel's product may miss the real-valued one by the fp32 error of the
        # sum (4e-6 of sum |vx| |w^|, the bound the standalone product is tested to) plus one rounding to binary16;
        # that times |r| (halved by div2), plus one spacing of the output's own rounding.
        f64 = np.float64
        sp = lambda v: np.exp2(np.floor(np.log2(np.maximum(np.abs(v), 2.0 ** -14))) - 10)  # binary16 spacing at |v|
        p_e = vx_g.astype(f64) @ vw.exact()
        mag = np.abs(vx_g.astype(f64)) @ np.abs(vw.exact())
        tol = (4e-6 * mag + sp(p_e)) * np.abs(r_g.astype(f64)) * (0.5 if div2 else 1.0) + sp(strict.astype(f64))
        err = np.abs(x_out.numpy().astype(f64) - strict.astype(f64))
        assert (err <= tol).all(), "x_out from kernel intermediates (uint8): worst %.2f of its bound" % float((err / tol).max())
        return
    out_g = po.gemm_f16(vx_g, vref, "f16")
    strict = np.array([po.lib.orc_hfma(int(a), int(b), int(c)) for a, b, c in
                       zip(out_g.view(np.uint16), r_g.view(np.uint16), x.view(np.uint16))], np.uint16).view(np.float16)
    if div2:
        strict = (strict.astype(np.float32) / 2).astype(np.float16)
    # (a product of F > 8192 terms is several times the residual it is added to: where the fp32 sum lands on the other
    # side of a rounding boundary than the exact sum, one spacing of the product is a few spacings of the output)
    assert_close_f16(x_out.numpy(), strict, max_ulp=1 if F_ <= 8192 else 4, max_frac=0.002, what="x_out from kernel intermediates")


@pytest.mark.parametrize("C_,H_", [(2560, 40), (512, 8), (5120, 80)])
@pytest.mark.parametrize("quant", [False, True])
def test_att_one_v5_1(C_, H_, quant):
    """kernels/cuda/att.cu:267-335,393-425 (serves RWKV-5.1 and 5.2)."""
    S_ = C_ // H_
    x, sx = h(rng.standard_normal(C_) * 2), h(rng.standard_normal(C_))
    s = rng.standard_normal((H_, S_, S_)).astype(np.float32)
    ln_w, ln_b = h(1 + 0.1 * rng.standard_normal(C_)), h(0.1 * rng.standard_normal(C_))
    lx_w = (1 + 0.1 * rng.standard_normal(C_)).astype(np.float32)
    lx_b = (0.1 * rng.standard_normal(C_)).astype(np.float32)
    mixes = [h(rng.uniform(0, 1, C_)) for _ in range(4)]
    td = np.exp(-np.exp(rng.uniform(-6, 0, (H_, S_)))).astype(np.float32)
    tf = rng.uniform(-1, 1, (H_, S_)).astype(np.float32)
    ws, refs = [], []
    for _ in range(5):
        w, r = make_weight(h(rng.standard_normal((C_, C_)) * 0.02), quant)
        ws.append(w)
        refs.append(r)
    if quant:  # the oracle's one-token products multiply the unrounded uint8 weights, as the kernels do
        for w, r in zip(ws, refs):
            po.register_u8(r, *w.parts)
    try:
        ref_x, ref_xx, ref_s = po.att_v5_2_f16(x, sx, s, ln_w, ln_b, lx_w, lx_b, *mixes, td, tf, *refs, H_)
    finally:
        for r in refs:
            po.unregister_u8(r)
    x_out, xx_out = DevBuf.empty(C_, np.float16), DevBuf.empty(C_, np.float16)
    s_out = DevBuf.empty((H_, S_, S_), np.float32)
    wsb = DevBuf(L().frhip_decode_workspace_bytes(C_, 4 * C_))
    fr.check(L().frhip_att_one_v5_1(C_, H_, keep(x).ptr, keep(sx).ptr, keep(s).ptr, keep(ln_w).ptr, keep(ln_b).ptr,
                                    keep(lx_w).ptr, keep(lx_b).ptr, *[keep(m).ptr for m in mixes], keep(td).ptr,
                                    keep(tf).ptr, *[w.ref for w in ws], x_out.ptr, xx_out.ptr, s_out.ptr, wsb.ptr,
                                    None))
    assert_close_f16(xx_out.numpy(), ref_xx, max_ulp=1, what="xx")
    assert np.allclose(s_out.numpy(), ref_s, rtol=1e-5, atol=2e-3 if quant else 1e-5)
    # groupnorm amplifies the fp32 summation-order noise of the head outputs; a few one-spacing
    # flips of the gated vector then spread over the output product
    # (and one layernorm output on the other side of a rounding boundary than the oracle's shifts every product a little)
    ln_flip = bool((xx_out.numpy() != ref_xx).any())
    # (the output product has C terms: at twice the width the same flips weigh more)
    loose = quant or ln_flip or C_ > 2560
    assert_close_f16(x_out.numpy(), ref_x, max_ulp=5 if loose else 3, max_frac=0.4 if loose else 0.2, what="x_out")


@pytest.mark.parametrize("C_,H_", [(2048, 32), (512, 8)])
@pytest.mark.parametrize("quant", [False, True])
def test_att_one_v5(C_, H_, quant):
    """RWKV-5.0, kernels/cuda/att.cu:219-265,362-391: no gate, one decay / bonus per head."""
    S_ = C_ // H_
    x, sx = h(rng.standard_normal(C_) * 2), h(rng.standard_normal(C_))
    s = rng.standard_normal((H_, S_, S_)).astype(np.float32)
    ln_w, ln_b = h(1 + 0.1 * rng.standard_normal(C_)), h(0.1 * rng.standard_normal(C_))
    lx_w = (1 + 0.1 * rng.standard_normal(C_)).astype(np.float32)
    lx_b = (0.1 * rng.standard_normal(C_)).astype(np.float32)
    mixes = [h(rng.uniform(0, 1, C_)) for _ in range(3)]
    td = np.exp(-np.exp(rng.uniform(-6, 0, H_))).astype(np.float32)
    tf = rng.uniform(-1, 1, H_).astype(np.float32)
    ws, refs = [], []
    for _ in range(4):
        w, r = make_weight(h(rng.standard_normal((C_, C_)) * 0.02), quant)
        ws.append(w)
        refs.append(r)
    ref_x, ref_xx, ref_s = po.att_v5_0_f16(x, sx, s, ln_w, ln_b, lx_w, lx_b, *mixes, td, tf, *refs, H_)
    x_out, xx_out = DevBuf.empty(C_, np.float16), DevBuf.empty(C_, np.float16)
    s_out = DevBuf.empty((H_, S_, S_), np.float32)
    wsb = DevBuf(L().frhip_decode_workspace_bytes(C_, 4 * C_))
    fr.check(L().frhip_att_one_v5(C_, H_, keep(x).ptr, keep(sx).ptr, keep(s).ptr, keep(ln_w).ptr, keep(ln_b).ptr,
                                  keep(lx_w).ptr, keep(lx_b).ptr, *[keep(m).ptr for m in mixes], keep(td).ptr,
                                  keep(tf).ptr, *[w.ref for w in ws], x_out.ptr, xx_out.ptr, s_out.ptr, wsb.ptr,
                                  None))
    assert_close_f16(xx_out.numpy(), ref_xx, max_ulp=1, what="xx")
    assert np.allclose(s_out.numpy(), ref_s, rtol=1e-5, atol=2e-3 if quant else 1e-5)
    assert_close_f16(x_out.numpy(), ref_x, max_ulp=5 if quant else 3, max_frac=0.4 if quant else 0.2, what="x_out")


@pytest.mark.parametrize("C_", [2048, 5120])  # 5120: the layernorm prologue loops over the vector
@pytest.mark.parametrize("quant", [False, True])
def test_head(quant, C_):
    V_ = 65536 if C_ == 2048 else 8192
    x, ln_w, ln_b = h(rng.standard_normal(C_) * 3), h(1 + 0.1 * rng.standard_normal(C_)), h(0.1 * rng.standard_normal(C_))
    V_ = 8192 if quant else V_
    hw, href = make_weight(h(rng.standard_normal((C_, V_)) * 0.02), quant)
    ref = po.gemm_f16(po.layernorm_f16(x, ln_w, ln_b), href, "f16").astype(np.float32)
    out = DevBuf.empty(V_, np.float32)
    fr.check(L().frhip_head(C_, keep(x).ptr, keep(ln_w).ptr, keep(ln_b).ptr, hw.ref, out.ptr, None))
    got = out.numpy()
    assert np.abs(got - ref).max() <= 2e-2
    if quant:  # tight against the real-valued weights, loose against the oracle's binary16 w^
        exact = po.layernorm_f16(x, ln_w, ln_b).astype(np.float64) @ hw.exact()
        # (the fp32 error of the factored sum, about 4e-6 of sum |x| |w^|, is comparable to half a spacing of these logits:
        # some land on the other side of a rounding boundary, none further than one spacing)
        assert_close_f16(got.astype(np.float16), exact.astype(np.float16), max_ulp=1, max_frac=0.15, what="logits vs real-valued weights")
        assert np.abs(got - ref).max() <= 4e-3
    else:
        assert_close_f16(got.astype(np.float16), ref.astype(np.float16), max_ulp=2, max_frac=0.05, what="logits")


def test_head_mirror_in_pinned_host_memory():
    """frhip_head_mirror stores every logit to a second buffer as well; with that buffer in pinned host
    memory the host reads, after a stream wait, exactly what the device buffer holds."""
    C_, V_ = 2048, 8192
    x, ln_w, ln_b = h(rng.standard_normal(C_) * 3), h(1 + 0.1 * rng.standard_normal(C_)), h(0.1 * rng.standard_normal(C_))
    hw, _ = make_weight(h(rng.standard_normal((C_, V_)) * 0.02), False)
    out = DevBuf.empty(V_, np.float32)
    hp = C.c_void_p()
    fr.check(L().frhip_host_malloc(C.byref(hp), 4 * V_))
    try:
        host = np.ctypeslib.as_array(C.cast(hp, C.POINTER(C.c_float)), shape=(V_,))
        host[:] = -1.0
        fr.check(L().frhip_head_mirror(C_, keep(x).ptr, keep(ln_w).ptr, keep(ln_b).ptr, hw.ref, out.ptr, hp, None))
        fr.check(L().frhip_device_sync())
        assert np.array_equal(host, out.numpy())
        ref = DevBuf.empty(V_, np.float32)
        fr.check(L().frhip_head(C_, keep(x).ptr, keep(ln_w).ptr, keep(ln_b).ptr, hw.ref, ref.ptr, None))
        assert np.array_equal(ref.numpy(), out.numpy())
    finally:
        fr.check(L().frhip_host_free(hp))


@pytest.mark.parametrize("quant", [False, True])
def test_greedy_decode_128_steps_matches_oracle(quant):
    """fp16 logits within max-abs 2e-2 of the oracle and the same greedy token over 128 steps
    (12 layers: two /2 rescales are crossed)."""
    L_, C_, F_, V_ = 12, 512, 2048, 4096
    params, emb = make_model(4, L_, C_, F_, V_, seed=5)
    hm = HipModelV4(L_, C_, F_, V_, params, emb, quant=quant)
    om = po.Model(4, po.F16, L_, C_, F_, 0, V_, params, emb, quant=hm.oracle_quant)
    prompt = np.random.default_rng(42).integers(0, V_, 16)
    worst, swaps = greedy_against_oracle(hm.run, om.run, prompt, 128, tol=2e-2, tag="12x512 quant=%s" % quant)
    print("quant", quant, "worst |dlogit|", worst, "near-tie swaps", swaps, flush=True)
    # states agree after 144 tokens
    for l in (0, 11):
        for j in (1, 2, 3):
            ref = om.state[l * 5 + j]
            assert np.abs(hm.state[l][j].numpy() - ref).max() <= 5e-3 * np.abs(ref).max()
    om.close()
    # ResetStates then rerun is bit-identical (tests/test_model.cpp:93-97)
    hm.reset()
    a = [hm.run(t).copy() for t in (1, 2, 3)]
    hm.reset()
    b = [hm.run(t).copy() for t in (1, 2, 3)]
    assert all(np.array_equal(x, y) for x, y in zip(a, b))


def test_one_layer_at_the_1b5_shape():
    """One layer of the 1.5B shape (C 2048, F 8192) plus the 65536-wide head, 4 tokens."""
    params, emb = make_model(4, 1, 2048, 8192, 65536, seed=9)
    hm = HipModelV4(1, 2048, 8192, 65536, params, emb)
    om = po.Model(4, po.F16, 1, 2048, 8192, 0, 65536, params, emb)
    for t in (0, 65535, 777, 777):
        lh, lo = hm.run(t), om.run(t)
        assert np.abs(lh - lo).max() <= 2e-2
