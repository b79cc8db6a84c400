"""GPU tests of the host layer's operator surface on the `hip` device beyond the fused model path:
the shape operators and silu the reference's own loops call (kernels/kernels.h:131,194,221,255), the
operator-by-operator seq loop written like kernels/default/model_forward_seq.cpp:105-183, the caching
allocator (the role of kernels/cuda/allocator.cpp:412-474), RWKV-5.1 dispatch, and state snapshots."""
import importlib
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import pyoracle as po
from hipref import greedy_against_oracle, same_token_or_near_tie
from synth import make_model

fr = importlib.import_module("faster-rwkv_amd")
rng = np.random.default_rng(2024)


@pytest.fixture(autouse=True)
def _rng_per_test(request):
    """Every test draws from a generator seeded by its own name, so its data do not depend on which
    other tests ran before it (or on cases added to them)."""
    import zlib
    global rng
    rng = np.random.default_rng([2024, zlib.crc32(request.node.name.encode())])

SLICE, CAT, TRANSPOSE, SILU = 0, 1, 2, 3


# ------------------------------------------------------------------ slice / cat / transpose / silu
def _np_slice(a, ranges):
    """Range semantics of kernels/cuda/slice.cu:54-66: (0,0,0) = whole dimension, negative start/end count
    from the end, extent (end - start) / interval."""
    idx = []
    for dim, (st, iv, en) in zip(a.shape, ranges):
        if (st, iv, en) == (0, 0, 0):
            st, iv, en = 0, 1, dim
        st, en = st + dim * (st < 0), en + dim * (en < 0)
        idx.append(slice(st, st + ((en - st) // iv) * iv, iv))
    return a[tuple(idx)]


@pytest.mark.parametrize("shape,ranges", [
    ((1024, 256), [(-1, 1, 1024), (0, 0, 0)]),      # the last row, model_forward_seq.cpp:171 (a view, no launch)
    ((77, 128), [(0, 1, -1), (0, 0, 0)]),           # all rows but the last: the token shift's xx[:-1]
    ((77, 128), [(5, 3, 70), (16, 2, -7)]),         # strided in both dimensions
    ((9, 7, 33), [(2, 1, 8), (0, 0, 0), (-20, 4, 33)]),
    ((2, 3, 4, 10), [(0, 0, 0), (1, 1, 3), (0, 2, 4), (3, 3, 10)]),
    ((640,), [(100, 7, 640)]),
])
@pytest.mark.parametrize("dtype", [np.float16, np.float32, np.int8])
def test_slice_follows_the_reference_range_semantics(shape, ranges, dtype):
    a = (rng.standard_normal(shape) * 50).astype(dtype)
    got = fr.shape_op(SLICE, a, params=[v for r in ranges for v in r])
    want = _np_slice(a, ranges)
    assert got.shape == want.shape and np.array_equal(got, want)


def test_slice_rejects_ranges_outside_the_tensor():
    a = np.zeros((8, 4), np.float32)
    for bad in ([(0, 1, 9), (0, 0, 0)], [(5, 1, 3), (0, 0, 0)], [(0, 0, 0), (0, -1, 4)], [(0, 0, 0), (-9, 1, 4)]):
        with pytest.raises(fr.FrhipError):
            fr.shape_op(SLICE, a, params=[v for r in bad for v in r])


@pytest.mark.parametrize("sa,sb,dim", [((1, 256), (63, 256), 0), ((5, 3), (5, 9), 1), ((2, 3, 4), (2, 5, 4), 1),
                                       ((2, 3, 4), (2, 3, 1), -1), ((16,), (3,), 0)])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_cat(sa, sb, dim, dtype):
    a, b = rng.standard_normal(sa).astype(dtype), rng.standard_normal(sb).astype(dtype)
    got = fr.shape_op(CAT, a, b, params=[dim])
    assert np.array_equal(got, np.concatenate([a, b], axis=dim))


@pytest.mark.parametrize("shape,da,db", [((64, 64), 0, 1), ((33, 130), 1, 0), ((40, 64, 64), 1, 2), ((40, 64, 64), -1, -2),
                                         ((3, 5, 7), 0, 2), ((2, 3, 4, 5), 1, 3)])
@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int8])
def test_transpose(shape, da, db, dtype):
    a = (rng.standard_normal(shape) * 40).astype(dtype)
    got = fr.shape_op(TRANSPOSE, a, params=[da, db])
    assert np.array_equal(got, np.swapaxes(a, da, db))


def test_silu_is_the_fused_path_arithmetic():
    """Every finite binary16 value: x / (1 + half(exp(-x))) in half (kernels/cuda/att.cu:145-152), which
    the oracle restates; fp32: x / (1 + exp(-x))."""
    bits = np.arange(65536, dtype=np.uint16)
    x = bits.view(np.float16).copy()
    x[~np.isfinite(x)] = 0
    got = fr.shape_op(SILU, x.reshape(256, 256))
    assert np.array_equal(got.view(np.uint16), po.silu_f16(x.reshape(256, 256)).view(np.uint16))
    xf = (rng.standard_normal(5000) * 4).astype(np.float32)
    want = xf.astype(np.float64) / (1 + np.exp(-xf.astype(np.float64)))
    assert np.allclose(fr.shape_op(SILU, xf), want, rtol=3e-6, atol=1e-7)
    assert abs(float(fr.shape_op(SILU, np.asarray([1.0], np.float32))[0]) - 0.7310586) < 1e-6  # not x / (1 - e^x)


# ------------------------------------------------------------------ the reference-shaped seq loop
def _write(tmp_path, version, name, L, C, F, V, H, seed):
    params, emb = make_model({"4": 4, "5": 50}.get(version, 52), L, C, F, V, H, seed=seed)
    path = str(tmp_path / name)
    fr.write_fr(path, version, L, C, F, H, params, emb)
    return path, params, emb


@pytest.mark.parametrize("version,H", [("5.2", 8), ("4", 0), ("5", 8)])
@pytest.mark.parametrize("strategy", ["hip fp16", "hip int8"])
def test_operator_by_operator_seq_loop_matches_the_fused_seq_forward(tmp_path, version, H, strategy):
    """FR_HIP_GENERIC=1 runs seq mode as the reference writes it (vgather, att_seq_*, ffn_seq, scalar_div_,
    slice + squeeze of the last row, layernorm, matmul, cast_dtype) through the registry.  The layer
    operators are the same launches as the fused forward's; the tail differs (layernorm and matmul as two
    launches instead of one), so logits agree to rounding, and the states left behind are the same."""
    path, _, _ = _write(tmp_path, version, "m.fr", 6, 512, 1792, 2048, H, seed=31)
    ids = [int(t) for t in np.random.default_rng(5).integers(0, 2048, 250)]
    m = fr.Model(path, strategy)
    fused = m.run(ids)
    fused_next = m.run(7)
    full = m.run_full(ids[:40])
    m.close()
    os.environ["FR_HIP_GENERIC"] = "1"
    try:
        g = fr.Model(path, strategy)
        generic = g.run(ids)
        generic_next = g.run(7)
        gfull = g.run_full(ids[:40])
        g.close()
    finally:
        del os.environ["FR_HIP_GENERIC"]
    assert np.abs(fused - generic).max() <= 4e-3 and same_token_or_near_tie(fused, generic)
    assert np.abs(fused_next - generic_next).max() <= 4e-3
    assert gfull.shape == full.shape and np.abs(full - gfull).max() <= 4e-3


# ------------------------------------------------------------------ RWKV-5.1
@pytest.mark.parametrize("strategy", ["hip fp16", "hip int8"])
def test_rwkv5_1_model_one_token_path_and_seq_fallback(tmp_path, strategy):
    """Version string "5.1": one-token steps take att_one_v5_1 like 5.2 (kernels/default/model_forward.cpp:138);
    upstream has no seq operator for it (model_forward_seq.cpp:127-128), seq mode is the loop of one-token steps."""
    from synth import matrix_indices, quantize_u8
    L, C, F, V, H = 6, 512, 1792, 2048, 8
    path, params, emb = _write(tmp_path, "5.1", "v51.fr", L, C, F, V, H, seed=33)
    qd = {i: quantize_u8(params[i]) for i in matrix_indices(52, L)} if strategy.endswith("int8") else None
    om = po.Model(52, po.F16, L, C, F, H, V, params, emb, quant=qd)
    m = fr.Model(path, strategy)
    worst, _ = greedy_against_oracle(m.run, om.run, [3, 1, 4, 1, 5], 48, tol=2e-2, tag="v5.1 " + strategy)
    m.reset()
    om.reset()
    prompt = [int(t) for t in np.random.default_rng(6).integers(0, V, 40)]
    ls = m.run(prompt)               # seq mode of a 5.1 model: one-token steps underneath
    for t in prompt:
        lo = om.run(t)
    assert np.abs(ls - lo).max() <= 2e-2 and same_token_or_near_tie(ls, lo)
    m.close()
    om.close()


# ------------------------------------------------------------------ state snapshots, owned logits
@pytest.mark.parametrize("version,H", [("4", 0), ("5.2", 4)])
def test_a_copy_of_states_is_a_snapshot_that_set_states_restores(tmp_path, version, H):
    """`auto s = model.states(); model.Run(...); model.set_states(s);` returns the model to the snapshot,
    as with the reference's operators, which return fresh state tensors every step
    (kernels/cuda/att.cu:344-353)."""
    path, _, _ = _write(tmp_path, version, "m.fr", 4, 256, 896, 1024, H, seed=35)
    m = fr.Model(path, "hip fp16")
    for t in (5, 6, 7):
        m.run(t)
    snap = m.snapshot()
    first = [m.run(t) for t in (8, 9, 10, 11)]
    m.restore(snap)
    again = [m.run(t) for t in (8, 9, 10, 11)]
    assert all(np.array_equal(a, b) for a, b in zip(first, again))
    # the snapshot is still intact after the second pass, and survives a seq-mode call as well
    m.run([1, 2, 3, 4, 5])
    m.restore(snap)
    third = [m.run(t) for t in (8, 9, 10, 11)]
    assert all(np.array_equal(a, b) for a, b in zip(first, third))
    # the greedy loop kept on the device moves to fresh buffers as well while a snapshot is held
    # (its graphs name the old ones), and gives the same tokens again from the restored state
    m.restore(snap)
    g1, _ = m.greedy(8, 37)
    after1 = m.run(3).copy()
    m.restore(snap)
    g2, _ = m.greedy(8, 37)
    after2 = m.run(3).copy()
    assert np.array_equal(g1, g2) and np.array_equal(after1, after2)
    m.restore(snap)
    t, want = 8, []
    for _ in range(37):
        t = int(np.argmax(m.run(t)))
        want.append(t)
    assert want == g1.tolist()
    m.free_snapshot(snap)
    m.close()


def test_owned_logits_mode_returns_the_same_logits(tmp_path):
    path, _, _ = _write(tmp_path, "4", "m.fr", 2, 256, 1024, 1024, 0, seed=37)
    m = fr.Model(path, "hip fp16")
    view_mode = [m.run(t) for t in (1, 2, 3)]
    toks, _ = m.greedy(1, 12)
    m.close()
    os.environ["FR_HIP_OWNED_LOGITS"] = "1"
    try:
        o = fr.Model(path, "hip fp16")
        owned = [o.run(t) for t in (1, 2, 3)]
        otoks, _ = o.greedy(1, 12)
        o.close()
    finally:
        del os.environ["FR_HIP_OWNED_LOGITS"]
    assert all(np.array_equal(a, b) for a, b in zip(view_mode, owned)) and np.array_equal(toks, otoks)


# ------------------------------------------------------------------ the caching allocator
def test_allocator_reuses_memory_and_decoding_makes_no_driver_calls():
    m = fr.Model("synthetic:v=4,L=4,C=512,F=2048,V=4096,seed=3", "hip fp16")
    m.greedy(1, 8)                      # warm-up: plan buffers, graph capture
    r0, u0, c0 = fr.allocator_stats()
    toks, _ = m.greedy(int(1), 64)
    r1, u1, c1 = fr.allocator_stats()
    assert c1 == c0, "decoding 64 tokens called the driver %d times" % (c1 - c0)
    assert (r1, u1) == (r0, u0)
    # prompts: the first T=1024 pass may grow the pool, the second must not
    ids = [int(t) for t in np.random.default_rng(1).integers(0, 4096, 1024)]
    m.run(ids)
    r2, u2, c2 = fr.allocator_stats()
    m.run(ids)
    r3, u3, c3 = fr.allocator_stats()
    assert (r3, c3) == (r2, c2), "a second prompt of the same length grew the pool"
    assert u3 == u2
    m.close()
    r4, u4, _ = fr.allocator_stats()
    assert u4 < u3 and r4 == r3         # the model's memory went back to the pool, not to the driver


def test_allocator_prompts_of_changing_length_are_served_from_the_first_ones_memory():
    """Large blocks are split for smaller requests and merge again when released
    (kernels/cuda/allocator.cpp:267-268, 449-459): after the longest prompt no later, shorter one
    makes the pool grow."""
    m = fr.Model("synthetic:v=4,L=4,C=1024,F=4096,V=4096,seed=5", "hip fp16")
    g = np.random.default_rng(2)
    m.run([int(t) for t in g.integers(0, 4096, 1024)])
    r0, u0, c0 = fr.allocator_stats()
    for T in (700, 333, 1000, 1024, 64, 1001):
        m.reset()
        m.run([int(t) for t in g.integers(0, 4096, T)])
        r, u, c = fr.allocator_stats()
        assert (r, c) == (r0, c0), "a prompt of %d tokens after one of 1024 grew the pool by %d bytes" % (T, r - r0)
    m.close()


def test_allocator_splits_large_blocks_and_merges_them_again():
    h = fr.host()
    fr.init()
    h.fr_allocator_trim()
    MB = 1 << 20
    big = h.fr_hip_alloc(64 * MB)
    assert big
    calls = fr.allocator_stats()[2]
    h.fr_hip_free(big)
    a = h.fr_hip_alloc(16 * MB)          # at least twice the request: the block is split, the front handed out
    b = h.fr_hip_alloc(16 * MB)          # from the tail
    c = h.fr_hip_alloc(30 * MB)          # the remaining 32 MiB are less than twice 30: handed out whole
    assert (a, b, c) == (big, big + 16 * MB, big + 32 * MB) and fr.allocator_stats()[2] == calls
    used = fr.allocator_stats()[1]
    h.fr_hip_free(b)                     # a hole between two live blocks
    assert fr.allocator_stats()[1] == used - 16 * MB
    d = h.fr_hip_alloc(10 * MB)          # best fit: the 16 MiB hole, not split (10 < 16 < 20)
    assert d == b and fr.allocator_stats()[1] == used
    for p in (a, c, d):
        h.fr_hip_free(p)
    again = h.fr_hip_alloc(64 * MB)      # the three blocks merged back into the segment
    assert again == big and fr.allocator_stats()[2] == calls
    h.fr_hip_free(again)
    # a segment with a live block is not released; once it is free as a whole, it is
    a = h.fr_hip_alloc(8 * MB)
    assert a == big
    reserved = fr.allocator_stats()[0]
    assert h.fr_allocator_trim() == 0 and fr.allocator_stats()[0] == reserved
    h.fr_hip_free(a)
    assert h.fr_allocator_trim() >= 64 * MB


def test_allocator_alignment_reuse_trim_and_out_of_memory():
    h = fr.host()
    fr.init()
    ptrs = [h.fr_hip_alloc(n) for n in (1, 511, 512, 513, 4096, 100_000, (1 << 20) + 1, 5 << 20)]
    assert all(p and p % 512 == 0 for p in ptrs)            # kernels/allocator.h:9-10
    assert len(set(ptrs)) == len(ptrs)
    _, used, calls = fr.allocator_stats()
    for p in ptrs:
        assert h.fr_hip_free(p) == 0
    _, used2, _ = fr.allocator_stats()
    assert used2 < used
    again = h.fr_hip_alloc(5 << 20)                          # served from the pool (best fit): no driver call
    assert again and again % 512 == 0 and fr.allocator_stats()[2] == calls
    h.fr_hip_free(again)
    # an absurd request fails as an error, not a crash, and the allocator goes on working
    assert not h.fr_hip_alloc(1 << 46)
    assert b"out of device memory" in h.fr_last_error()
    p = h.fr_hip_alloc(3 << 20)
    assert p and p % 512 == 0
    h.fr_hip_free(p)
    # Trim gives the cached large blocks back to the driver (the refused request above already emptied
    # the cache once, as the allocator's last resort before it reports failure)
    reserved = fr.allocator_stats()[0]
    freed = h.fr_allocator_trim()
    assert freed >= (3 << 20) and fr.allocator_stats()[0] == reserved - freed
    assert h.fr_allocator_trim() == 0
    # releasing a pointer the allocator never handed out is reported, not fatal
    assert h.fr_hip_free(12345 * 512) == 0
