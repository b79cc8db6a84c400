"""GPU parity tests of the primitive operators, through the C ABI, against the oracle."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import pyoracle as po
from hipref import DevBuf, L, PackedWeight, assert_close_f16, dev, fr, make_weight

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


rng = np.random.default_rng(123)


@pytest.fixture(autouse=True)
def _rng_per_test(request):
    """Every test draws from a generator seeded by its own name, so its data do not depend on which
    other tests ran before it (or on cases added to them)."""
    import zlib
    global rng
    rng = np.random.default_rng([123, zlib.crc32(request.node.name.encode())])


def h(x):
    return np.asarray(x, np.float32).astype(np.float16)


def test_runtime_identifies_gfx950_and_roundtrips_memory():
    fr.init()
    name = C.create_string_buffer(128)
    cus, mem = C.c_int(), C.c_size_t()
    fr.check(L().frhip_device_info(name, 128, C.byref(cus), C.byref(mem)))
    print("device:", name.value.decode(), cus.value, "CUs", mem.value >> 30, "GiB", flush=True)
    assert b"gfx950" in name.value and cus.value >= 200
    a = rng.integers(0, 255, 100003).astype(np.uint8)
    assert np.array_equal(keep(a).numpy(), a)


def test_known_answer_fill_then_scalar_div():
    """tests/test_ops.cpp:9-16"""
    x = DevBuf.empty(256, np.float16)
    fr.check(L().frhip_fill(x.ptr, fr.F16, 1.0, 256, None))
    fr.check(L().frhip_scalar_div_f16(x.ptr, 2.0, 256, None))
    y = DevBuf.empty(256, np.float32)
    fr.check(L().frhip_cast(x.ptr, fr.F16, y.ptr, fr.F32, 256, None))
    assert (y.numpy() == np.float32(0.5)).all()


@pytest.mark.parametrize("K,N,dt", [(64, 64, np.float16), (130, 70, np.float16), (257, 1000, np.uint8), (2048, 512, np.uint8)])
def test_pack_transpose(K, N, dt):
    a = rng.integers(0, 60000 if dt == np.float16 else 255, (K, N)).astype(np.uint16 if dt == np.float16 else np.uint8)
    src, dst = keep(a), DevBuf.empty((N, K), a.dtype)
    fr.check(L().frhip_pack_transpose(src.ptr, dst.ptr, K, N, a.dtype.itemsize, None))
    assert np.array_equal(dst.numpy(), a.T)


def test_cast_roundtrip_and_rtne():
    x = (rng.standard_normal(5000) * 10).astype(np.float32)
    a, b = keep(x), DevBuf.empty(5000, np.float16)
    fr.check(L().frhip_cast(a.ptr, fr.F32, b.ptr, fr.F16, 5000, None))
    assert np.array_equal(b.numpy().view(np.uint16), po.f2h(x).view(np.uint16))


@pytest.mark.parametrize("rows,cols", [(1, 2048), (7, 768), (3, 2560), (33, 96)])
def test_layernorm_f16(rows, cols):
    x, g, b = h(rng.standard_normal((rows, cols)) * 3), h(1 + 0.1 * rng.standard_normal(cols)), h(0.1 * rng.standard_normal(cols))
    y = DevBuf.empty((rows, cols), np.float16)
    fr.check(L().frhip_layernorm(keep(x).ptr, keep(g).ptr, keep(b).ptr, y.ptr, rows, cols, fr.F16, None))
    assert_close_f16(y.numpy(), po.layernorm_f16(x, g, b), max_ulp=1, what="layernorm")


def test_layernorm_f32_and_groupnorm():
    x = rng.standard_normal((5, 2560)).astype(np.float32)
    g, b = rng.standard_normal(2560).astype(np.float32), rng.standard_normal(2560).astype(np.float32)
    y = DevBuf.empty((5, 2560), np.float32)
    fr.check(L().frhip_layernorm(keep(x).ptr, keep(g).ptr, keep(b).ptr, y.ptr, 5, 2560, fr.F32, None))
    assert np.allclose(y.numpy(), po.layernorm_f32(x, g, b), atol=2e-5, rtol=1e-5)
    fr.check(L().frhip_groupnorm_f32(keep(x).ptr, 40, keep(g).ptr, keep(b).ptr, y.ptr, 5, 2560, None))
    assert np.allclose(y.numpy(), po.groupnorm_f32(x, 40, g, b), atol=2e-5, rtol=1e-5)


def test_dequant_all_codes_bit_exact():
    """Every code 0..255 against a grid of binary16 scale patterns, bit for bit."""
    K, N = 256, 64
    q = np.arange(256, dtype=np.uint8)[:, None].repeat(N, axis=1)
    mxs = h([-0.09, -0.031, 0.0, 0.0123, -1.7, 3e-5, -0.5, 2.0])
    rxs = h([0.17, 0.011, 1.0, 0.33, 5.5, 1e-3, 0.0625, 2.5e-4])
    mx, rx = np.tile(mxs, 8), np.repeat(rxs, 8)
    for my_v, ry_v in [(-0.07, 0.93), (0.0, 1.0), (0.011, 0.5), (-2.0, 0.031), (6e-5, 0.999)]:
        my, ry = np.full(K, my_v, np.float16), np.full(K, ry_v, np.float16)
        ref = po.dequant_u8(q, mx, rx, my, ry)  # [K,N]
        w = PackedWeight(q=q, mx=mx, rx=rx, my=my, ry=ry)
        out = DevBuf.empty((N, K), np.float16)
        fr.check(L().frhip_dequant_u8(w.ref, out.ptr, None))
        assert np.array_equal(out.numpy().T.view(np.uint16), ref.view(np.uint16))
        # the matrix-vector kernel evaluates the same formula in fp32 without the final rounding of
        # w^ to binary16: a one-hot activation returns q c ry + mx + my of row k to fp32 accuracy
        y = DevBuf.empty(N, np.float32)
        f = np.float64
        for k in (0, 1, 17, 200, 255):
            e = np.zeros(K, np.float16)
            e[k] = 1
            fr.check(L().frhip_gemv(keep(e).ptr, w.ref, y.ptr, fr.F32, None))
            terms = (np.abs(q[k].astype(f) * (rx.astype(f) / 255) * f(ry[k])), np.abs(mx.astype(f)), abs(f(my[k])))
            exact = q[k].astype(f) * (rx.astype(f) / 255) * f(ry[k]) + mx.astype(f) + f(my[k])
            assert (np.abs(y.numpy() - exact) <= 4e-7 * (terms[0] + terms[1] + terms[2]) + 1e-30).all(), k


@pytest.mark.parametrize("K,N", [(2048, 320), (2560, 100), (36, 7)])  # 16 codes per thread; K % 16 != 0: 4 per thread
def test_dequant_random_matrix_bit_exact(K, N):
    from synth import quantize_u8
    w = h(rng.standard_normal((K, N)) * 0.02)
    q, mx, rx, my, ry = quantize_u8(w)
    pw = PackedWeight(q=q, mx=mx, rx=rx, my=my, ry=ry)
    out = DevBuf.empty((N, K), np.float16)
    fr.check(L().frhip_dequant_u8(pw.ref, out.ptr, None))
    assert np.array_equal(out.numpy().T.view(np.uint16), po.dequant_u8(q, mx, rx, my, ry).view(np.uint16))


# K above 9216 (binary16) / 16384 (uint8): rows consumed in slices
@pytest.mark.parametrize("K,N", [(2048, 2048), (2048, 8192), (8192, 2048), (2560, 2560), (8960, 2560), (768, 50277), (64, 3), (16, 1),
                                 (10240, 2560), (16384, 515), (20480, 130), (32768, 9), (9232, 33)])
@pytest.mark.parametrize("quant", [False, True])
def test_gemv_against_oracle(K, N, quant):
    x = h(rng.standard_normal(K))
    w = h(rng.standard_normal((K, N)) * 0.02)
    pw, wref = make_weight(w, quant)
    ref32 = po.gemm_f16(x, wref, "f32")
    y32, y16 = DevBuf.empty(N, np.float32), DevBuf.empty(N, np.float16)
    fr.check(L().frhip_gemv(keep(x).ptr, pw.ref, y32.ptr, fr.F32, None))
    fr.check(L().frhip_gemv(keep(x).ptr, pw.ref, y16.ptr, fr.F16, None))
    tol = 2e-6 * np.sqrt(K) * np.abs(ref32).max() + 1e-6
    if not quant:
        assert np.abs(y32.numpy() - ref32).max() <= tol + 2e-5
        assert_close_f16(y16.numpy(), ref32.astype(np.float16), max_ulp=1, what="gemv f16 out")
        return
    # uint8: the kernel evaluates sum_k x_k (q c ry + mx + my) in fp32 without rounding w^ to
    # binary16 -> tight against the real-valued formula in float64 ...
    exact = x.astype(np.float64) @ pw.exact()
    mag = np.abs(x.astype(np.float64)) @ np.abs(pw.exact())
    assert (np.abs(y32.numpy() - exact) <= 4e-6 * mag + 1e-6).all()
    # ... and within the w^-rounding noise of the oracle, which multiplies by binary16 w^
    # (relative error up to 2^-12 per element, uniform): eight standard deviations of that sum
    rms = lambda a: float(np.sqrt(np.mean(np.asarray(a, np.float64) ** 2)))
    noise = 8 * (2.0 ** -12 / np.sqrt(3)) * np.sqrt(K) * rms(x) * rms(wref)
    assert np.abs(y32.numpy() - ref32).max() <= tol + noise + 2e-5
    r16 = ref32.astype(np.float16).astype(np.float32)
    half_spacing = np.exp2(np.floor(np.log2(np.maximum(np.abs(r16), 1e-7))) - 11)
    assert (np.abs(y16.numpy().astype(np.float32) - r16) <= noise + 2 * half_spacing).all()


def test_gemv_rejects_bad_arguments():
    w = PackedWeight(w_kn=h(rng.standard_normal((64, 8))))
    y = DevBuf.empty(8, np.float32)
    x = keep(h(np.zeros(64)))
    assert L().frhip_gemv(None, w.ref, y.ptr, fr.F32, None) == -1
    assert L().frhip_gemv(x.ptr, w.ref, y.ptr, 7, None) == -1
    bad = fr.Weight(w.c.data, None, None, None, None, 60, 8, fr.F16)
    assert L().frhip_gemv(x.ptr, C.byref(bad), y.ptr, fr.F32, None) == -2
    assert b"multiple of 16" in L().frhip_error_string()


def test_argmax_first_of_ties():
    x = rng.standard_normal(65536).astype(np.float32)
    x[[1234, 40000]] = 9.0
    out = DevBuf.empty(1, np.int32)
    fr.check(L().frhip_argmax_f32(keep(x).ptr, 65536, out.ptr, None))
    assert out.numpy()[0] == 1234 == po.lib.orc_argmax(x.ctypes.data_as(C.c_void_p), 65536)


@pytest.mark.parametrize("n,nblocks", [(65536, 64), (65529, 64), (1000, 64), (7, 3), (4096, 1)])
def test_argmax_blocks_first_of_ties(n, nblocks):
    """Per-slice {value, index} pairs, reduced as the host does (greater value, then smaller index),
    give the oracle's arg-max: ragged lengths, slices that are short or empty, ties within a slice,
    across slices and across the groups of four a thread scans."""
    x = rng.standard_normal(n).astype(np.float32)
    ties = sorted({n // 3, n // 3 + 1, n // 2, n - 1})
    x[ties] = 9.0
    pairs = DevBuf.empty(2 * nblocks, np.float32)
    fr.check(L().frhip_argmax_blocks_f32(keep(x).ptr, n, pairs.ptr, nblocks, None))
    raw = pairs.numpy()
    # the two-destination form stores the same pairs twice
    first, second = DevBuf.empty(2 * nblocks, np.float32), DevBuf.empty(2 * nblocks, np.float32)
    fr.check(L().frhip_argmax_blocks_f32_mirror(keep(x).ptr, n, first.ptr, second.ptr, nblocks, None))
    assert first.numpy().tobytes() == raw.tobytes() == second.numpy().tobytes()
    vals, idxs = raw[0::2], raw[1::2].view(np.int32)
    best, at = -np.inf, n
    for v, i in zip(vals, idxs):
        if v > best or (v == best and i < at):
            best, at = v, int(i)
    assert at == ties[0] == po.lib.orc_argmax(x.ctypes.data_as(C.c_void_p), n) and best == 9.0
    ln = ((n + nblocks - 1) // nblocks + 3) // 4 * 4
    for b in range(nblocks):  # every pair describes its own slice
        sl = x[b * ln:min((b + 1) * ln, n)]
        if len(sl):
            assert vals[b] == sl.max() and idxs[b] == b * ln + int(np.argmax(sl))
        else:
            assert vals[b] == -np.inf and idxs[b] == n


def _host_rule(vals, idxs, n_rows):
    """hip::ModelForward's second step of the arg-max (greater value, then smaller index; nothing
    finite found: token 0)."""
    best, at = -np.inf, n_rows
    for v, i in zip(vals, idxs):
        if v > best or (v == best and i < at):
            best, at = v, int(i)
    return at if at < n_rows else 0


@pytest.mark.parametrize("case", ["random", "ties_across_slices", "all_minus_inf", "nan_slices", "nothing_found", "one_pair"])
def test_embed_argmax_follows_the_host_rule(case):
    """frhip_embed_argmax: the token picked from the per-slice pairs is the one the host's reduction
    picks, it is noted in ids[counter % ids_len], the counter advances and the token's row is copied;
    two calls in a row use two slots."""
    n_rows, row = 1000, 256
    tab = h(rng.standard_normal((n_rows, row)))
    npairs = 1 if case == "one_pair" else 64
    vals = rng.standard_normal(npairs).astype(np.float32)
    idxs = rng.permutation(n_rows)[:npairs].astype(np.int32)
    if case == "ties_across_slices":
        vals[[5, 17, 40]] = 7.5
    elif case == "all_minus_inf":
        vals[:] = -np.inf
    elif case == "nan_slices":
        vals[::2] = np.nan
    elif case == "nothing_found":  # what argmax_blocks reports for slices without a finite maximum
        vals[:] = -np.inf
        idxs[:] = n_rows
    want = _host_rule(vals, idxs, n_rows)
    if case == "ties_across_slices":
        assert want == int(min(idxs[[5, 17, 40]]))
    if case == "nothing_found":
        assert want == 0
    raw = np.empty(2 * npairs, np.float32)
    raw[0::2] = vals
    raw[1::2] = idxs.view(np.float32)
    ids = DevBuf.empty(8, np.int32)
    fr.check(L().frhip_fill(ids.ptr, fr.F32, 0.0, 8, None))
    counter = keep(np.array([13], np.uint32))  # slot 13 % 8 = 5, then 6
    out = DevBuf.empty(row, np.float16)
    for call in range(2):
        fr.check(L().frhip_embed_argmax(keep(tab).ptr, n_rows, 2 * row, keep(raw).ptr, npairs, ids.ptr, 8, counter.ptr,
                                        out.ptr, None))
        assert np.array_equal(out.numpy(), tab[want])
        assert counter.numpy()[0] == 14 + call
    got = ids.numpy()
    assert got[5] == want and got[6] == want and not got[[0, 1, 2, 3, 4, 7]].any()


def test_gather_rows():
    tab = h(rng.standard_normal((1000, 256)))
    ids = np.array([5, 999, 0, 5, 123], np.int32)
    out = DevBuf.empty((5, 256), np.float16)
    fr.check(L().frhip_gather_rows(keep(tab).ptr, keep(ids).ptr, out.ptr, 5, 512, None))
    assert np.array_equal(out.numpy(), tab[ids])
