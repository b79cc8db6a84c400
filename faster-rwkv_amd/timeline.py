"""Per-wave timeline of the row-streaming decode kernel (csrc/decode.hip, rows_kernel).

Needs the measurement build of the library, in which every wave notes the 100 MHz clock at eleven points and leaves
the notes in device memory when it ends:

    make -C faster-rwkv_amd/csrc timeline
    FRHIP_LIBRARY=faster-rwkv_amd/libfrhip_timeline.so python3 faster-rwkv_amd/timeline.py fp16|int8 [n_embd ffn]

The script replays one token of a 4-layer RWKV-4 model of the given width (default 2048 / 8192, random weights,
vocabulary 65536) as a graph, as the model's forward pass does, and prints for the last att_out, ffn_front and ffn_out
launch (the attention front has a kernel of its own, without notes) when, counted from the first wave's entry, the
waves reached each point: median, earliest and latest wave, in microseconds.
"""
import ctypes as C
import importlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
fr = importlib.import_module("faster-rwkv_amd")

POINTS = ["entry", "prologue operands requested", "first rows requested", "normalised (x arrived, 2 reductions)",
          "staged, at the barrier", "through the barrier", "all rows requested (uint8: sums gathered)", "",
          "products done", "reduced", "epilogue issued", "", "", "", "", "stores done"]


def main():
    u8 = len(sys.argv) > 1 and sys.argv[1] == "int8"
    C_ = int(sys.argv[2]) if len(sys.argv) > 2 else 2048
    F_ = int(sys.argv[3]) if len(sys.argv) > 3 else 8192
    L_, V_ = 4, 65536
    lib = fr.lib()
    if not hasattr(lib, "frhip_timeline_read"):
        raise SystemExit("this library was built without FRHIP_TIMELINE: make -C faster-rwkv_amd/csrc timeline, "
                         "then set FRHIP_LIBRARY to faster-rwkv_amd/libfrhip_timeline.so")
    fr.init()
    rng = np.random.default_rng(0)
    keep = []

    def dev(a):
        b = fr.DevBuf.from_numpy(a)
        keep.append(b)
        return b

    def weight(K, N):
        if u8:
            d = dev(rng.integers(0, 255, (N, K), dtype=np.uint8))
            sc = [dev(rng.uniform(0.01, 0.02, n).astype(np.float16)) for n in (N, N, K, K)]
            return fr.Weight(d.ptr, sc[0].ptr, sc[1].ptr, sc[2].ptr, sc[3].ptr, K, N, fr.U8)
        d = dev((rng.standard_normal((N, K), dtype=np.float32) * 0.02).astype(np.float16))
        return fr.Weight(d.ptr, None, None, None, None, K, N, fr.F16)

    h = lambda a: np.asarray(a, np.float32).astype(np.float16)
    layers = []
    for _ in range(L_):
        layers.append(dict(
            vec=[dev(h(np.ones(C_))), dev(h(np.zeros(C_)))] + [dev(h(rng.uniform(0, 1, C_))) for _ in range(3)],
            td=dev((-np.exp(rng.uniform(-5, 1, C_))).astype(np.float32)), tf=dev(rng.uniform(-1, 1, C_).astype(np.float32)),
            att=[weight(C_, C_) for _ in range(4)],
            fvec=[dev(h(np.ones(C_))), dev(h(np.zeros(C_)))] + [dev(h(rng.uniform(0, 1, C_))) for _ in range(2)],
            ffn=[weight(C_, F_), weight(F_, C_), weight(C_, C_)],
            st=[dev(h(np.zeros(C_))), dev(np.zeros(C_, np.float32)), dev(np.zeros(C_, np.float32)),
                dev(np.full(C_, -1e30, np.float32)), dev(h(np.zeros(C_)))],
            xx=[dev(h(np.zeros(C_))), dev(h(np.zeros(C_)))]))
    ln_o = [dev(h(np.ones(C_))), dev(h(np.zeros(C_)))]
    head = weight(C_, V_)
    x = dev(h(rng.standard_normal(C_)))
    logits = fr.DevBuf.empty(V_, np.float32)
    ws = fr.DevBuf(lib.frhip_decode_workspace_bytes(C_, F_))
    st = C.c_void_p()
    fr.check(lib.frhip_stream_create(C.byref(st)))

    def token():
        for v in layers:
            s = v["st"]
            fr.check(lib.frhip_att_one_v4(C_, x.ptr, s[0].ptr, s[1].ptr, s[2].ptr, s[3].ptr, *[t.ptr for t in v["vec"]],
                                          v["td"].ptr, v["tf"].ptr, *[C.byref(w) for w in v["att"]], x.ptr,
                                          v["xx"][0].ptr, s[1].ptr, s[2].ptr, s[3].ptr, ws.ptr, st))
            fr.check(lib.frhip_ffn_one(C_, F_, x.ptr, s[4].ptr, *[t.ptr for t in v["fvec"]],
                                       *[C.byref(w) for w in v["ffn"]], x.ptr, v["xx"][1].ptr, 0, ws.ptr, st))
        fr.check(lib.frhip_head(C_, x.ptr, ln_o[0].ptr, ln_o[1].ptr, C.byref(head), logits.ptr, st))

    # one capture = one set of launches; each took the slot its launch number names, and every replay overwrites it
    fr.check(lib.frhip_graph_begin(st))
    token()
    g = C.c_void_p()
    fr.check(lib.frhip_graph_end(st, C.byref(g)))
    for _ in range(5):
        fr.check(lib.frhip_graph_launch(g, st))
    fr.check(lib.frhip_stream_sync(st))
    lib.frhip_timeline_read.argtypes = [C.c_void_p, C.POINTER(C.c_int)]
    lib.frhip_timeline_read.restype = C.c_int
    buf = np.zeros((8, 4096, 16), np.uint64)
    cnt = C.c_int()
    fr.check(lib.frhip_timeline_read(buf.ctypes.data, C.byref(cnt)), "frhip_timeline_read")
    per_token = 3 * L_ + 1  # row-kernel launches of the token: att_out, ffn_front, ffn_out per layer, then the head
    slot_of = {}
    for i in range(per_token):  # later launches overwrite earlier ones
        slot_of[(cnt.value - per_token + i) % 8] = ["att_out", "ffn_front", "ffn_out", "head"][i % 3 if i < 3 * L_ else 3]
    print("%s weights, n_embd %d, ffn %d; microseconds after the launch's first wave entered" % ("uint8" if u8 else "binary16", C_, F_))
    for slot, name in sorted(slot_of.items(), key=lambda kv: kv[1]):
        if name == "head":
            continue
        t = buf[slot].astype(np.float64) * 0.01
        t = t[t[:, 0] > 0]
        t0 = t[:, 0].min()
        print("== %s: %d waves, last wave entered at %.2f, last stores done at %.2f" % (name, len(t), t[:, 0].max() - t0, t[:, 15].max() - t0))
        for i in [1, 2, 3, 4, 5, 6, 8, 9, 10, 15]:
            col = t[:, i][t[:, i] > 0] - t0
            if len(col):
                print("   %-42s median %5.2f   first %5.2f   last %5.2f" % (POINTS[i], np.median(col), col.min(), col.max()))


if __name__ == "__main__":
    main()
