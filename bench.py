#!/usr/bin/env python3
"""Headline benchmark: batch-1 greedy decode of an RWKV-4 1.5B-shaped model on one MI355X.

    python bench.py [--gpus 1] [--steps 512] [--warmup 16] [--dtype fp16|int8]

A "step" is one decoded token of the loop the reference's chat.cpp:56-92 / bench_model.cpp:7-8 run: one
rwkv::Model::Run(id) through the `hip` device (fused kernels replayed as a HIP graph) that returns the fp32
logits on the host, the greedy choice of the next token, the next Run -- one host wait per token
(FR_HIP_GREEDY_ON_HOST=1).  The same loop kept on the device (fr_greedy_decode's default, which the reference's
API does not have) is reported beside it in `extra`.  Weights are random-init of
the named architecture (there are no checkpoints here) and are resident in HBM before the
timed region starts.

Prints ONE JSON line.  Besides the decode rate it carries
  roofline     -- the row-streaming matrix-vector kernels (all of their launches in one
                  token): algorithmic bytes / summed launch time, measured with HIP events on
                  the launch stream, against the 8 TB/s HBM peak;
  cpu_baseline -- the CPU oracle's fp32 path (oracle/, a port: the reference has no CPU model
                  path) timed on this host on a bounded sample of the same workload.
"""
import argparse
import ctypes as C
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBS = 8000.0

CONFIGS = {
    # BASELINE.json configs[1] / configs[2]
    "fp16": dict(workload="rwkv4-1.5B-shaped fp16 decode bs1 (24 layers, d_model 2048, ffn 8192, vocab 65536)",
                 spec="synthetic:v=4,L=24,C=2048,F=8192,V=65536,seed=1236", strategy="hip fp16", wbytes=2),
    "int8": dict(workload="rwkv4-1.5B-shaped uint8 decode bs1 (24 layers, d_model 2048, ffn 8192, vocab 65536)",
                 spec="synthetic:v=4,L=24,C=2048,F=8192,V=65536,seed=1237", strategy="hip int8", wbytes=1),
}
L_, C_, F_, V_ = 24, 2048, 8192, 65536

# HBM bytes per token (fetched + written) by hardware counters, and the profile that records the runs
TRAFFIC = {
    "fp16": (2915.2e6 + 2.3e6, "profiles/decode_rwkv4_1b5_fp16_hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE; "
                                "not re-read in this run)"),
    "int8": (1503.8e6 + 2.3e6, "profiles/decode_rwkv4_1b5_int8_hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE; "
                                "not re-read in this run)"),
}


def algorithmic_bytes_per_token(wbytes):
    """Bytes the matrix-vector kernels must move per token: every matrix weight once, plus
    (uint8) its offsets/ranges, plus the activation vector in and the result out."""
    mats = [(C_, C_)] * 4 + [(C_, F_), (F_, C_), (C_, C_)]
    per_layer = 0
    for k, n in mats:
        per_layer += k * n * wbytes + 2 * k + 2 * n
        if wbytes == 1:
            per_layer += 4 * (k + n)
    head = C_ * V_ * wbytes + 2 * C_ + 4 * V_ + (4 * (C_ + V_) if wbytes == 1 else 0)
    return L_ * per_layer + head


def measure_kernels(fr, cfg, reps=20):
    """Time the launches of one token with HIP events recorded on the launch stream itself:
    total time of the fused kernels (they are back to back on one stream, so the events
    bracket exactly their execution), averaged over `reps` tokens after a warm-up."""
    lib = fr.lib()
    fr.init()
    rng = np.random.default_rng(0)
    u8 = cfg["wbytes"] == 1
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
            vec=[dev(h(np.ones(C_))), dev(h(np.zeros(C_))), dev(h(rng.uniform(0, 1, C_))), dev(h(rng.uniform(0, 1, C_))),
                 dev(h(rng.uniform(0, 1, C_)))],
            td=dev((-np.exp(rng.uniform(-5, 1, C_))).astype(np.float32)), tf=dev(rng.uniform(-1, 1, C_).astype(np.float32)),
            att=[weight(C_, C_) for _ in range(4)],
            fvec=[dev(h(np.ones(C_))), dev(h(np.zeros(C_))), dev(h(rng.uniform(0, 1, C_))), dev(h(rng.uniform(0, 1, C_)))],
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
        for l, v in enumerate(layers):
            s = v["st"]
            fr.check(lib.frhip_att_one_v4(C_, x.ptr, s[0].ptr, s[1].ptr, s[2].ptr, s[3].ptr, *[t.ptr for t in v["vec"]],
                                          v["td"].ptr, v["tf"].ptr, *[C.byref(w) for w in v["att"]], x.ptr,
                                          v["xx"][0].ptr, s[1].ptr, s[2].ptr, s[3].ptr, ws.ptr, st))
            fr.check(lib.frhip_ffn_one(C_, F_, x.ptr, s[4].ptr, *[t.ptr for t in v["fvec"]],
                                       *[C.byref(w) for w in v["ffn"]], x.ptr, v["xx"][1].ptr,
                                       1 if (l + 1) % 6 == 0 else 0, ws.ptr, st))
        fr.check(lib.frhip_head(C_, x.ptr, ln_o[0].ptr, ln_o[1].ptr, C.byref(head), logits.ptr, st))

    fr.check(lib.frhip_graph_begin(st))
    token()
    g = C.c_void_p()
    fr.check(lib.frhip_graph_end(st, C.byref(g)))
    e0, e1 = C.c_void_p(), C.c_void_p()
    lib.frhip_event_create(C.byref(e0))
    lib.frhip_event_create(C.byref(e1))
    for _ in range(3):
        fr.check(lib.frhip_graph_launch(g, st))
    fr.check(lib.frhip_stream_sync(st))
    fr.check(lib.frhip_event_record(e0, st))
    for _ in range(reps):
        fr.check(lib.frhip_graph_launch(g, st))
    fr.check(lib.frhip_event_record(e1, st))
    fr.check(lib.frhip_event_sync(e1))
    ms = C.c_float()
    fr.check(lib.frhip_event_elapsed_ms(e0, e1, C.byref(ms)))
    lib.frhip_graph_destroy(g)
    lib.frhip_stream_destroy(st)
    n_launch = 4 * L_ + 1
    return ms.value / reps, n_launch


def probe_bandwidth(fr, nbytes=2 << 30, reps=5):
    """Read-only and copy ceilings of this GPU as seen by plain streaming kernels (GB/s)."""
    lib = fr.lib()
    fr.init()
    src, dst = fr.DevBuf(nbytes), fr.DevBuf(nbytes)
    sink = fr.DevBuf(1 << 16)
    fr.check(lib.frhip_memset_async(src.ptr, 1, nbytes, None))
    st = C.c_void_p()
    fr.check(lib.frhip_stream_create(C.byref(st)))
    e0, e1 = C.c_void_p(), C.c_void_p()
    lib.frhip_event_create(C.byref(e0))
    lib.frhip_event_create(C.byref(e1))
    out = {}
    for name, fn, traffic in (("read", lambda: lib.frhip_read_probe(src.ptr, nbytes, sink.ptr, st), nbytes),
                              ("copy", lambda: lib.frhip_copy_probe(dst.ptr, src.ptr, nbytes, st), 2 * nbytes)):
        fr.check(fn())
        fr.check(lib.frhip_stream_sync(st))
        fr.check(lib.frhip_event_record(e0, st))
        for _ in range(reps):
            fr.check(fn())
        fr.check(lib.frhip_event_record(e1, st))
        fr.check(lib.frhip_event_sync(e1))
        ms = C.c_float()
        fr.check(lib.frhip_event_elapsed_ms(e0, e1, C.byref(ms)))
        out[name + "_GBs"] = round(traffic * reps / (ms.value * 1e-3) / 1e9, 1)
    lib.frhip_stream_destroy(st)
    return out


def prompt_only(fr, T):
    """One prompt length alone (profiling aid): best of 4 passes over T tokens of the fp16 model."""
    cfg = CONFIGS["fp16"]
    m = fr.Model(cfg["spec"], cfg["strategy"])
    ids = np.random.default_rng(43).integers(0, V_, T)
    best = 1e9
    for _ in range(4):
        m.reset()
        t0 = time.perf_counter()
        m.run(ids)
        best = min(best, time.perf_counter() - t0)
    m.close()
    return {"prompt_len": T, "prompt_ms": round(best * 1e3, 3), "prompt_tok_s": round(T / best, 1)}


def prefill_extra(fr):
    """BASELINE configuration 4: T=1024 seq-mode prefill of the same fp16 model."""
    cfg = CONFIGS["fp16"]
    m = fr.Model(cfg["spec"], cfg["strategy"])
    ids = np.random.default_rng(43).integers(0, V_, 1024)
    best = 1e9
    for _ in range(4):
        m.reset()
        t0 = time.perf_counter()
        m.run(ids)
        best = min(best, time.perf_counter() - t0)
    # a short prompt of the same model (its products are split over K across the compute units that 64-row tiles leave idle)
    short = 1e9
    for _ in range(4):
        m.reset()
        t0 = time.perf_counter()
        m.run(ids[:64])
        short = min(short, time.perf_counter() - t0)
    m.close()
    flops = 2.0 * 1024 * L_ * 54525952
    return {"prefill_T1024_tok_s": round(1024 / best, 1), "prefill_ms": round(best * 1e3, 3), "prefill_T64_ms": round(short * 1e3, 3),
            "prefill_gemm_TFLOPs_over_whole_pass": round(flops / best / 1e12, 1),
            "prefill_frac_of_2500_TFLOPs": round(flops / best / 2.5e15, 4)}


def rwkv5_extra(fr):
    """BASELINE configuration 5: RWKV-5.2 3B-shaped uint8 model, T=512 seq-mode prefill then 256
    greedy one-token steps."""
    m = fr.Model("synthetic:v=5.2,L=32,C=2560,F=8960,V=65536,H=40,seed=1238", "hip int8")
    ids = np.random.default_rng(44).integers(0, V_, 512)
    best = 1e9
    os.environ["FR_HIP_SEQ_IMAGE"] = "0"  # the default: the uint8 weights expanded to binary16 per call, nothing kept
    try:
        for _ in range(3):
            m.reset()
            t0 = time.perf_counter()
            lg = m.run(ids)
            best = min(best, time.perf_counter() - t0)
    finally:
        del os.environ["FR_HIP_SEQ_IMAGE"]
    os.environ["FR_HIP_GREEDY_ON_HOST"] = "1"  # Model::Run per token, as the headline
    try:
        m.greedy(int(np.argmax(lg)), 16)
        _, secs = m.greedy(17, 256)
    finally:
        del os.environ["FR_HIP_GREEDY_ON_HOST"]
    # the same prompt with the binary16 image of the uint8 weights kept on the device (FR_HIP_SEQ_IMAGE=1, opt-in:
    # 2 more bytes per weight, no expansion per call); the first pass makes the images and is not timed
    os.environ["FR_HIP_SEQ_IMAGE"] = "1"
    try:
        kept = 1e9
        for i in range(4):
            m.reset()
            t0 = time.perf_counter()
            lg2 = m.run(ids)
            if i:
                kept = min(kept, time.perf_counter() - t0)
    finally:
        del os.environ["FR_HIP_SEQ_IMAGE"]
    assert np.array_equal(lg, lg2), "kept binary16 image changed the logits"
    m.close()
    # Algorithmic bytes per token: the uint8 codes of every matrix once, their offsets / ranges, the [H, 64, 64] fp32
    # state of every layer read and written, activation vectors in and out.
    C5, F5, Lr = 2560, 8960, 32
    mats = [(C5, C5)] * 5 + [(C5, F5), (F5, C5), (C5, C5)]
    per_layer = sum(k * n + 4 * (k + n) + 2 * k + 2 * n for k, n in mats) + 2 * 4 * C5 * 64
    abytes = Lr * per_layer + C5 * V_ + 4 * (C5 + V_) + 2 * C5 + 4 * V_
    return {"rwkv5_3b_int8_prefill_T512_ms": round(best * 1e3, 2), "rwkv5_3b_int8_prefill_tok_s": round(512 / best, 1),
            "rwkv5_3b_int8_prefill_T512_kept_fp16_image_ms": round(kept * 1e3, 2),
            "rwkv5_3b_int8_decode_tok_s": round(256 / secs, 1),
            "rwkv5_3b_int8_decode_bytes_per_token": abytes,
            "rwkv5_3b_int8_decode_GBs": round(abytes * 256 / secs / 1e9, 1),
            "rwkv5_3b_int8_decode_frac_of_hbm_peak": round(abytes * 256 / secs / 1e9 / HBM_PEAK_GBS, 4)}


def cpu_baseline(seconds_budget=20.0):
    """The oracle's fp32 one-token forward on the host cores (OpenMP over output columns): the whole
    24-layer 1.5B shape (6 GB of fp32 weights; every layer has weight arrays of its own, filled from one
    random block, so that no layer finds its weights in a cache), greedy tokens, for a bounded number of
    tokens -- on all threads the runtime gives, and on one."""
    import pyoracle as po
    rng = np.random.default_rng(1)

    def mat(k, n):
        return (rng.standard_normal((k, n), dtype=np.float32) * 0.02)

    def vec(lo, hi):
        return rng.uniform(lo, hi, C_).astype(np.float32)

    block = [np.ones(C_, np.float32), np.zeros(C_, np.float32), vec(0, 1), vec(0, 1), vec(0, 1),
             -np.exp(vec(-5, 1)), vec(-1, 1), mat(C_, C_), mat(C_, C_), mat(C_, C_), mat(C_, C_),
             np.ones(C_, np.float32), np.zeros(C_, np.float32), vec(0, 1), vec(0, 1), mat(C_, F_), mat(F_, C_),
             mat(C_, C_)]
    params = []
    for _ in range(L_):
        params += [a.copy() for a in block]
    params += [np.ones(C_, np.float32), np.zeros(C_, np.float32), mat(C_, V_)]
    emb = rng.standard_normal((1024, C_), dtype=np.float32)
    model = po.Model(4, po.F32, L_, C_, F_, 0, V_, params, emb)

    def per_token(budget, most):
        tok = int(np.argmax(model.run(1))) % 1024
        n, t0 = 0, time.perf_counter()
        while True:
            tok = int(np.argmax(model.run(tok))) % 1024
            n += 1
            dt = time.perf_counter() - t0
            if dt > budget or n >= most:
                return dt / n, n

    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    t_all, n_all = per_token(seconds_budget * 0.5, 128)
    # the same on one thread (the oracle's loops are OpenMP-parallel: the thread count is the runtime's to set)
    gomp = C.CDLL("libgomp.so.1")
    gomp.omp_set_num_threads(1)
    try:
        t_one, n_one = per_token(seconds_budget * 0.5, 8)
    finally:
        gomp.omp_set_num_threads(cores)
    return {"value": round(1.0 / t_all, 3), "unit": "tok/s", "cores": cores, "kind": "port",
            "single_thread_value": round(1.0 / t_one, 3), "nproc": os.cpu_count(),
            "sample": "oracle fp32 one-token forward of the whole 24-layer 1.5B shape (vocab 65536), greedy: "
                      "%d tokens timed on %d threads, %d tokens on one thread" % (n_all, cores, n_one)}


def probe_mfma(fr, iters=20000, reps=3):
    """What the matrix cores of this GPU sustain on nothing but v_mfma_f32_32x32x16_f16 (register operands,
    no memory traffic), with all-zero and with random operands: TFLOP/s from HIP events and the core clock
    each wave saw (core-clock ticks / 100 MHz ticks of its loop)."""
    import numpy as np
    lib = fr.lib()
    fr.init()
    name = C.create_string_buffer(128)
    cus = C.c_int()
    fr.check(lib.frhip_device_info(name, 128, C.byref(cus), None))
    st = C.c_void_p()
    fr.check(lib.frhip_stream_create(C.byref(st)))
    e0, e1 = C.c_void_p(), C.c_void_p()
    lib.frhip_event_create(C.byref(e0))
    lib.frhip_event_create(C.byref(e1))
    rng = np.random.default_rng(0)
    out = {"compute_units": cus.value, "mfma_per_wave": iters * 6}
    for waves in (4, 8):
        sink = fr.DevBuf(cus.value * waves * 64 * 4)
        clocks = fr.DevBuf.empty((cus.value * waves, 2), np.uint64)
        for label, data in (("zero", np.zeros((4096, 2, 8), np.float16)),
                            ("random", rng.standard_normal((4096, 2, 8)).astype(np.float16))):
            ops = fr.DevBuf.from_numpy(data)
            fr.check(lib.frhip_mfma_probe(waves, iters, ops.ptr, sink.ptr, clocks.ptr, st))
            fr.check(lib.frhip_stream_sync(st))
            best = 1e9
            for _ in range(reps):
                fr.check(lib.frhip_event_record(e0, st))
                fr.check(lib.frhip_mfma_probe(waves, iters, ops.ptr, sink.ptr, clocks.ptr, st))
                fr.check(lib.frhip_event_record(e1, st))
                fr.check(lib.frhip_event_sync(e1))
                ms = C.c_float()
                fr.check(lib.frhip_event_elapsed_ms(e0, e1, C.byref(ms)))
                best = min(best, ms.value)
            ck = clocks.numpy().astype(np.float64)
            flop = cus.value * waves * iters * 6 * 32768.0
            out["%dwaves_%s" % (waves, label)] = {"ms": round(best, 3), "TFLOPs": round(flop / (best * 1e-3) / 1e12, 1),
                                                  "core_clock_MHz": round(float(np.median(ck[:, 0] / ck[:, 1])) * 100.0, 0)}
    lib.frhip_stream_destroy(st)
    return out


_GEMM_SHAPES = ((2048, 6144), (2048, 8192), (2048, 10240), (2048, 2048), (8192, 2048))

_TORCH_YARDSTICK = r"""
import json, sys, torch
T, reps = int(sys.argv[1]), int(sys.argv[2])
out = {}
for K, N in %s:
    nrot = max(2, int(600e6 // (K * N * 2)))
    tw = [torch.randn(N, K, device="cuda", dtype=torch.float16) * 0.02 for _ in range(nrot)]
    tx = torch.randn(T, K, device="cuda", dtype=torch.float16)
    for w in tw:
        tx @ w.t()
    torch.cuda.synchronize()
    best = 1e9
    for _ in range(reps):
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        for w in tw:
            tx @ w.t()
        t1.record()
        torch.cuda.synchronize()
        best = min(best, t0.elapsed_time(t1) * 1e3 / nrot)
    out["%%dx%%dx%%d" %% (T, K, N)] = round(best, 1)
    del tw, tx
print(json.dumps(out))
""" % (repr(_GEMM_SHAPES),)


def probe_gemm(fr, T=1024, reps=4):
    """The prompt pass's matrix x matrix products one at a time (frhip_gemm, binary16 in and out, no epilogue), on
    weights that come from HBM (a rotation of matrices larger than the caches), and -- as a yardstick, not as
    part of the product -- torch.matmul (hipBLASLt / rocBLAS) on the same shapes and operand layout.  torch brings
    a HIP runtime of its own, so it runs in a child process, before this process touches the GPU."""
    import subprocess
    yard = {}
    try:
        r = subprocess.run([sys.executable, "-c", _TORCH_YARDSTICK, str(T), str(reps)], capture_output=True, text=True, timeout=300)
        yard = json.loads(r.stdout.strip().splitlines()[-1]) if r.returncode == 0 else {}
    except Exception as e:  # no torch, no GPU for it: the yardstick column stays empty
        print("[bench] torch yardstick not available: %r" % (e,), file=sys.stderr)
    lib = fr.lib()
    fr.init()
    rng = np.random.default_rng(0)
    e0, e1 = C.c_void_p(), C.c_void_p()
    lib.frhip_event_create(C.byref(e0))
    lib.frhip_event_create(C.byref(e1))
    out = {"T": T, "shapes": {}}
    for K, N in _GEMM_SHAPES:
        nrot = max(2, int(600e6 // (K * N * 2)))
        x = fr.DevBuf.from_numpy(rng.standard_normal((T, K)).astype(np.float16))
        w_nk = (rng.standard_normal((N, K)) * 0.02).astype(np.float16)  # output-major, as the kernels read weights
        ws = [fr.DevBuf.from_numpy(w_nk) for _ in range(nrot)]
        y = fr.DevBuf(T * N * 2)
        structs = [fr.Weight(w.ptr, None, None, None, None, K, N, fr.F16) for w in ws]

        def run():
            for wt in structs:
                fr.check(lib.frhip_gemm(x.ptr, C.byref(wt), y.ptr, T, fr.F16, None))
        run()
        fr.check(lib.frhip_device_sync())
        best = 1e9
        for _ in range(reps):
            fr.check(lib.frhip_event_record(e0, None))
            run()
            fr.check(lib.frhip_event_record(e1, None))
            fr.check(lib.frhip_event_sync(e1))
            ms = C.c_float()
            fr.check(lib.frhip_event_elapsed_ms(e0, e1, C.byref(ms)))
            best = min(best, ms.value * 1e3 / nrot)
        key = "%dx%dx%d" % (T, K, N)
        row = {"frhip_gemm_us": round(best, 1), "frhip_gemm_TFLOPs": round(2.0 * T * K * N / best * 1e-6, 0)}
        if key in yard:
            row["torch_matmul_us"] = yard[key]
            row["torch_matmul_TFLOPs"] = round(2.0 * T * K * N / yard[key] * 1e-6, 0)
        out["shapes"][key] = row
        del ws, structs, x, y
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=512)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--dtype", choices=["fp16", "int8"], default="fp16")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the int8-decode and prefill side measurements")
    ap.add_argument("--probe", action="store_true", help="only run the read/copy bandwidth probes and print them")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="only run the matrix-core rate probe (zero vs random operands) and print it")
    ap.add_argument("--gemm-probe", action="store_true",
                    help="only time the prompt pass's products standalone, beside torch.matmul on the same shapes, and print that")
    ap.add_argument("--prefill-only", action="store_true",
                    help="only run the T=1024 seq-mode prefill side measurement and print it (profiling aid)")
    ap.add_argument("--prompt-len", type=int, default=0,
                    help="only run a prompt of this many tokens through the fp16 model and print its time (profiling aid)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this backend runs batch-1 decode on ONE GPU; --gpus %d is not supported "
                 "(no multi-GPU path exists or is measured)" % args.gpus)
    if int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: launched with WORLD_SIZE > 1; only a single rank is supported")

    fr = importlib.import_module("faster-rwkv_amd")
    if args.probe:
        print(json.dumps(probe_bandwidth(fr)), flush=True)
        return
    if args.mfma_probe:
        print(json.dumps(probe_mfma(fr)), flush=True)
        return
    if args.gemm_probe:
        print(json.dumps(probe_gemm(fr)), flush=True)
        return
    if args.prompt_len > 0:
        print(json.dumps(prompt_only(fr, args.prompt_len)), flush=True)
        return
    if args.prefill_only:
        print(json.dumps(prefill_extra(fr)), flush=True)
        return
    cfg = CONFIGS[args.dtype]
    t0 = time.perf_counter()
    model = fr.Model(cfg["spec"], cfg["strategy"])
    build_s = time.perf_counter() - t0
    print("[bench] model built in %.1f s: %s" % (build_s, cfg["workload"]), file=sys.stderr, flush=True)

    # the timed loop: Model::Run per token with the host between the tokens
    os.environ["FR_HIP_GREEDY_ON_HOST"] = "1"
    try:
        model.greedy(0, 2)  # set-up, like the build: the first call captures the plan's graphs
        model.greedy(0, args.warmup)
        fr.check(fr.lib().frhip_device_sync())
        toks, secs = model.greedy(17, args.steps)
        fr.check(fr.lib().frhip_device_sync())
    finally:
        del os.environ["FR_HIP_GREEDY_ON_HOST"]
    # the same tokens with the greedy choice kept on the device (no host between the tokens)
    model.reset()
    model.greedy(0, 2)
    model.greedy(0, args.warmup)
    toks_dev, secs_dev = model.greedy(17, args.steps)
    fr.check(fr.lib().frhip_device_sync())
    model.close()
    assert np.array_equal(toks, toks_dev), "the device-side greedy chain chose other tokens than the loop of Run calls"
    ms_per_step = 1e3 * secs / args.steps
    tok_s = args.steps / secs

    kernel_ms, n_launch = measure_kernels(fr, cfg)
    abytes = algorithmic_bytes_per_token(cfg["wbytes"])
    achieved = abytes / (kernel_ms * 1e-3) / 1e9
    # HBM bytes per launch (average over the launches of one token) from the FETCH_SIZE / WRITE_SIZE
    # hardware counters, scaled by a copy kernel of known size.  Counters cannot be read inside this
    # run: the figures are those of the rocprofv3 --pmc runs of this command recorded in the named
    # profile (they change only when the kernels' access pattern does) and are labelled as such.
    traffic_bytes_per_token, traffic_source = TRAFFIC[args.dtype]
    traffic = round(traffic_bytes_per_token / n_launch) if traffic_bytes_per_token else None
    out = {
        "metric": "decode tok/s (RWKV-4 1.5B-shaped, bs1, greedy)", "value": round(tok_s, 2), "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16" if args.dtype == "fp16" else "u8 weights, f16 activations, f32 accumulate",
        "data": "synthetic (random-init weights, greedy token ids)",
        "config": {"workload": cfg["workload"], "strategy": cfg["strategy"], "steps": args.steps,
                   "host_loop": "Model::Run per token (chat.cpp:56-92, bench_model.cpp:7-8): one graph launch and one stream wait per "
                                "token, the logits in host memory after every token, the greedy token from the 64 per-slice arg-max "
                                "pairs the graph leaves beside them (extra.*_device_side_greedy_chain: the same tokens with the choice "
                                "kept on the device, the host waiting once per batch of tokens)"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": "row-streaming matrix-vector kernels (att_front/att_out/ffn_front/ffn_out/head), "
                               "%d launches per token" % n_launch,
                     "bytes_per_token": abytes, "kernel_ms_per_token": round(kernel_ms, 4),
                     "avg_launch_us": round(1e3 * kernel_ms / n_launch, 3)},
        "roofline_tok_s": round(1.0 / (abytes / (HBM_PEAK_GBS * 1e9)), 1),
    }
    dev_chain = {args.dtype + "_decode_tok_s_device_side_greedy_chain": round(args.steps / secs_dev, 2)}
    if args.no_extras:
        out["extra"] = dev_chain
    if not args.no_extras:
        extra = dict(dev_chain)
        other = "int8" if args.dtype == "fp16" else "fp16"
        ocfg = CONFIGS[other]
        om = fr.Model(ocfg["spec"], ocfg["strategy"])
        os.environ["FR_HIP_GREEDY_ON_HOST"] = "1"
        try:
            om.greedy(0, args.warmup)
            _, osecs = om.greedy(17, args.steps)
        finally:
            del os.environ["FR_HIP_GREEDY_ON_HOST"]
        om.reset()
        om.greedy(0, args.warmup)
        _, osecs_dev = om.greedy(17, args.steps)
        om.close()
        okms, _ = measure_kernels(fr, ocfg)
        ob = algorithmic_bytes_per_token(ocfg["wbytes"])
        extra[other + "_decode_tok_s"] = round(args.steps / osecs, 2)
        extra[other + "_decode_tok_s_device_side_greedy_chain"] = round(args.steps / osecs_dev, 2)
        extra[other + "_gemv_GBs"] = round(ob / (okms * 1e-3) / 1e9, 1)
        extra[other + "_gemv_frac_of_hbm_peak"] = round(ob / (okms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)
        # companions of the headline: the same loop over 512 steps when the run was shorter, and with
        # Model::Run returning a tensor of its own (FR_HIP_OWNED_LOGITS=1) instead of a view of pinned memory
        if args.dtype == "fp16":
            os.environ["FR_HIP_GREEDY_ON_HOST"] = "1"
            try:
                if args.steps < 512:
                    lm = fr.Model(cfg["spec"], cfg["strategy"])
                    lm.greedy(0, 16)
                    _, lsecs = lm.greedy(17, 512)
                    lm.close()
                    extra["fp16_decode_tok_s_512_steps"] = round(512 / lsecs, 2)
                os.environ["FR_HIP_OWNED_LOGITS"] = "1"
                wm = fr.Model(cfg["spec"], cfg["strategy"])
                wm.greedy(0, 16)
                _, wsecs = wm.greedy(17, 512)
                wm.close()
            finally:
                os.environ.pop("FR_HIP_OWNED_LOGITS", None)
                del os.environ["FR_HIP_GREEDY_ON_HOST"]
            extra["fp16_decode_tok_s_owned_logits"] = round(512 / wsecs, 2)
        extra.update(prefill_extra(fr))
        extra.update(rwkv5_extra(fr))
        extra.update(probe_bandwidth(fr))
        out["extra"] = extra
    out["cpu_baseline"] = None if args.no_cpu_baseline else cpu_baseline()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
