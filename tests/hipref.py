"""Test-side helpers: drive the HIP kernels through the C ABI (ctypes) on numpy data."""
import ctypes as C
import importlib

import numpy as np

fr = importlib.import_module("faster-rwkv_amd")
DevBuf, PackedWeight = fr.DevBuf, fr.PackedWeight


def L():
    return fr.lib()


def dev(a):
    return DevBuf.from_numpy(a)


def ulp_diff_f16(a, b):
    """Distance in units of binary16 representable values (monotone integer mapping)."""
    def key(x):
        u = np.asarray(x, np.float16).view(np.uint16).astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u)
    return np.abs(key(a) - key(b))


def assert_close_f16(got, ref, max_ulp=2, max_frac=0.03, what="", floor_rms=0.25):
    """|got-ref| <= max_ulp binary16 spacings, the spacing taken at max(|ref|, rms(ref)/4):
    an output formed by cancellation (x + out close to 0) inherits the absolute rounding
    error of its operands, which is not small in units of its own tiny spacing.  floor_rms
    raises that floor for outputs whose operands are larger than the output itself (the
    ffn product can be several times the residual it is added to)."""
    got, ref = np.asarray(got, np.float16), np.asarray(ref, np.float16)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    g32, r32 = got.astype(np.float32), ref.astype(np.float32)
    assert np.isfinite(g32).all(), what + ": non-finite output"
    floor = floor_rms * float(np.sqrt(np.mean(r32.astype(np.float64) ** 2))) + 1e-6
    mag = np.maximum(np.abs(r32), floor)
    spacing = np.exp2(np.floor(np.log2(mag)) - 10)
    err = np.abs(g32 - r32)
    bad = err > max_ulp * spacing
    assert not bad.any(), "%s: %d elements beyond %d spacings (worst %.2f)" % (
        what, bad.sum(), max_ulp, float((err / spacing).max()))
    assert (got.view(np.uint16) != ref.view(np.uint16)).mean() <= max_frac, "%s: %.3f of elements differ" % (
        what, (got.view(np.uint16) != ref.view(np.uint16)).mean())


def same_token_or_near_tie(lh, lo):
    """The greedy tokens agree, or the oracle's own margin between the two candidates is at most twice the
    largest logit difference of this step: a difference of d can swap two logits that lie less than 2d
    apart (one binary16 spacing at the top of a flat distribution is enough)."""
    th, to = int(np.argmax(lh)), int(np.argmax(lo))
    return th == to or float(lo[to] - lo[th]) <= 2 * float(np.abs(lh - lo).max())


def binary16_spacing(v):
    """Distance between neighbouring binary16 values at magnitude |v| (normal range)."""
    return float(np.exp2(np.floor(np.log2(max(abs(float(v)), 2.0 ** -14))) - 10))


class StateSynchronised:
    """A second `hip` model that is handed the oracle's recurrent state before every token, so that a step's
    comparison measures what ONE step of the implementation adds: two binary16 pipelines that are not
    bit-identical drift apart over many steps whatever the size of their first difference, and a free-running
    comparison cannot tell that drift from an implementation error.  `per_layer` = state tensors per layer
    (model.cpp:152-175: five for RWKV-4, three for RWKV-5)."""

    def __init__(self, model, oracle_model, per_layer):
        self.m, self.om, self.per = model, oracle_model, per_layer

    def run(self, tok):
        """Load the oracle's current state, then one token.  Call BEFORE the oracle runs the same token."""
        for i, a in enumerate(self.om.state):
            self.m.set_state(i // self.per, i % self.per, a)
        return self.m.run(int(tok))


def greedy_against_oracle(run_hip, run_oracle, prompt, steps, tol=2e-2, report=None, tag="", synced=None,
                          max_swaps=None, stats=None):
    """The parity criterion: feed `prompt` token by token, then `steps` greedy steps.

    Free-running (`run_hip`): at every step the logits agree within `tol` (max-abs; None = not asserted here) and
    the greedy tokens agree or differ at a near-tie (same_token_or_near_tie; both sides then continue with the
    oracle's token); at most `max_swaps` such steps.

    State-synchronised (`synced`, a StateSynchronised): the criterion as written, strictly -- at every step
    max-abs <= 2e-2 and the same greedy token whenever the oracle's margin between its two largest logits
    exceeds one binary16 spacing of the largest (logits are binary16 values: closer than that is a tie).

    Returns (worst free-running max-abs difference, free-running steps with unequal tokens); `stats`, if given,
    receives the state-synchronised figures as well."""
    import time
    st = stats if stats is not None else {}
    st.update(worst=0.0, swaps=0, sync_worst=0.0, sync_unequal=0, sync_steps=0)

    def one(tok):
        ls = synced.run(tok) if synced is not None else None  # before the oracle moves its state
        return run_hip(int(tok)), run_oracle(int(tok)), ls

    for t in prompt:
        lh, lo, ls = one(t)
    t0 = time.time()
    for step in range(steps):
        d = float(np.abs(lh - lo).max())
        st["worst"] = max(st["worst"], d)
        th, to = int(np.argmax(lh)), int(np.argmax(lo))
        if th != to:
            assert same_token_or_near_tie(lh, lo), "%s: greedy token differs at step %d (hip %d, oracle %d, oracle margin %g, |dlogit| %g)" % (
                tag, step, th, to, float(lo[to] - lo[th]), d)
            st["swaps"] += 1
        if ls is not None:
            ds = float(np.abs(ls - lo).max())
            st["sync_worst"] = max(st["sync_worst"], ds)
            st["sync_steps"] += 1
            assert ds <= 2e-2, "%s: state-synchronised step %d: |dlogit| %g" % (tag, step, ds)
            ts = int(np.argmax(ls))
            if ts != to:
                margin = float(lo[to] - np.partition(lo, -2)[-2])
                assert margin <= binary16_spacing(lo[to]), "%s: state-synchronised step %d: token %d, oracle %d, oracle margin %g" % (
                    tag, step, ts, to, margin)
                st["sync_unequal"] += 1
        lh, lo, ls = one(to)
        if report and step % 32 == 31:
            report("%s: %d steps, worst |dlogit| %.2e, %d near-tie swaps%s, %.0f s" % (
                tag, step + 1, st["worst"], st["swaps"],
                "; state-synchronised: worst %.2e, %d ties" % (st["sync_worst"], st["sync_unequal"]) if synced is not None else "",
                time.time() - t0))
    if tol is not None:
        assert st["worst"] <= tol, "%s: worst |dlogit| %g" % (tag, st["worst"])
    limit = max(1, steps // 16) if max_swaps is None else max_swaps
    assert st["swaps"] <= limit, "%s: tokens differed at %d of %d steps (limit %d)" % (tag, st["swaps"], steps, limit)
    return st["worst"], st["swaps"]


def make_weight(w_kn, quant=False):
    """PackedWeight from a [K,N] half matrix; quant=True quantises to uint8 first and
    also returns the oracle's dequantised [K,N] half matrix."""
    if not quant:
        return PackedWeight(w_kn=w_kn), np.ascontiguousarray(w_kn, np.float16)
    import pyoracle as po
    from synth import quantize_u8
    q, mx, rx, my, ry = quantize_u8(w_kn)
    pw = PackedWeight(q=q, mx=mx, rx=rx, my=my, ry=ry)
    pw.parts = (q, mx, rx, my, ry)
    f = np.float64
    # the real-valued formula the codes stand for, before any rounding of w^
    pw.exact = lambda: (q.astype(f) * (rx.astype(f) / 255)[None, :] * ry.astype(f)[:, None]
                        + mx.astype(f)[None, :] + my.astype(f)[:, None])
    return pw, po.dequant_u8(q, mx, rx, my, ry)


class HipModelV4:
    """RWKV-4 one-token forward assembled from the fused C-ABI operators, in the order of
    kernels/default/model_forward.cpp:105-188.  Parameters in the reference's positional order."""

    def __init__(self, L_, C_, F_, V_, params, emb, quant=False):
        self.L, self.C, self.F, self.V = L_, C_, F_, V_
        self.mats = {}
        self.oracle_params = list(params)
        self.oracle_quant = {}  # parameter index -> (q, mx, rx, my, ry): pyoracle.Model(..., quant=)
        self.p = []
        mat_pos = set()
        for l in range(L_):
            mat_pos |= {l * 18 + j for j in (7, 8, 9, 10, 15, 16, 17)}
        mat_pos.add(L_ * 18 + 2)
        for i, a in enumerate(params):
            if i in mat_pos:
                w, deq = make_weight(a, quant)
                self.p.append(w)
                self.oracle_params[i] = deq
                if quant:
                    self.oracle_quant[i] = w.parts
            else:
                self.p.append(dev(a))
        self.emb = dev(emb)
        self.emb_np = emb
        self.ws = DevBuf(L().frhip_decode_workspace_bytes(C_, F_))
        self.x = [DevBuf.empty(C_, np.float16) for _ in range(2)]
        self.logits = DevBuf.empty(V_, np.float32)
        self.reset()

    def reset(self):
        C_ = self.C
        self.state = []
        for _ in range(self.L):
            self.state.append([dev(np.zeros(C_, np.float16)), dev(np.zeros(C_, np.float32)),
                               dev(np.zeros(C_, np.float32)), dev(np.full(C_, -1e30, np.float32)),
                               dev(np.zeros(C_, np.float16))])
        self.spare = [dev(np.zeros(C_, np.float16)), dev(np.zeros(C_, np.float16))]

    def run(self, tok):
        lib, C_, F_ = L(), self.C, self.F
        fr.check(lib.frhip_memcpy(self.x[0].ptr, self.emb.ptr + int(tok) * C_ * 2, C_ * 2, fr.D2D))
        x = self.x[0]
        for l in range(self.L):
            p = self.p[l * 18:(l + 1) * 18]
            st = self.state[l]
            fr.check(lib.frhip_att_one_v4(C_, x.ptr, st[0].ptr, st[1].ptr, st[2].ptr, st[3].ptr,
                                          p[0].ptr, p[1].ptr, p[2].ptr, p[3].ptr, p[4].ptr, p[5].ptr, p[6].ptr,
                                          p[7].ref, p[8].ref, p[9].ref, p[10].ref,
                                          x.ptr, self.spare[0].ptr, st[1].ptr, st[2].ptr, st[3].ptr,
                                          self.ws.ptr, None), "att")
            st[0], self.spare[0] = self.spare[0], st[0]
            fr.check(lib.frhip_ffn_one(C_, F_, x.ptr, st[4].ptr, p[11].ptr, p[12].ptr, p[13].ptr, p[14].ptr,
                                       p[15].ref, p[16].ref, p[17].ref, x.ptr, self.spare[1].ptr,
                                       1 if (l + 1) % 6 == 0 else 0, self.ws.ptr, None), "ffn")
            st[4], self.spare[1] = self.spare[1], st[4]
        t = self.p[self.L * 18:]
        fr.check(lib.frhip_head(C_, x.ptr, t[0].ptr, t[1].ptr, t[2].ref, self.logits.ptr, None), "head")
        return self.logits.numpy()
