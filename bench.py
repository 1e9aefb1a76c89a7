#!/usr/bin/env python3
"""
Benchmark of the NervanaGPU compute core on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W        -> ONE JSON line on stdout
    python bench.py --all [--out FILE]                    -> also a per-case table
                                                             (GEMM, conv, pool, elementwise)

A "step" is one pass over benchmark configuration 2: the fp16 fully-connected GEMM sweep
with minibatch 128 ((M,K) in {(4096,9216),(4096,4096),(1000,4096)} x nn/nt/tn x
relu off/on x nearest/stochastic rounding), the square 4096^3 fp16 GEMM and the
batched 32 x 512^3 GEMM, with every operand already resident in HBM.  `value` is
the algorithmic flops of one step divided by its wall time.

`roofline` describes the dominant kernel of the step (the 4096^3 fp16 GEMM,
MFMA bound): algorithmic flops per launch / average launch duration measured
with HIP events on the launch stream.  `cpu_baseline` times the numpy oracle
(np.dot, the reference's own CPU check) on a bounded sample of the same step on
the host cores of the GPU box.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0     # dense fp16 MFMA, MI355X
PEAK_FP32_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0

FC_SHAPES = [(4096, 9216), (4096, 4096), (1000, 4096)]
MINIBATCH = 128


def fc_mnk(op, M, K, N=MINIBATCH):
    """op <-> fully-connected role (benchmarks/cublas.py:68-71 of the reference)"""
    if op == "nn":
        return M, N, K        # fprop  W(M,K) . x(K,N)
    if op == "tn":
        return K, N, M        # bprop  W(M,K)^T . d(M,N)
    return M, K, N            # update d(M,N) . x(K,N)^T


class GemmCase(object):
    def __init__(self, ng, op, m, n, k, relu=False, sr=False, dtype=np.float16, batch=0, seed=1):
        rng = np.random.default_rng(seed)
        self.op, self.m, self.n, self.k, self.relu, self.sr, self.batch = op, m, n, k, relu, sr, batch
        self.dtype = dtype
        bshape = (batch,) if batch else ()
        a_shape = bshape + ((k, m) if op[0] == "t" else (m, k))
        b_shape = bshape + ((n, k) if op[1] == "t" else (k, n))
        self.hA = rng.uniform(-1, 1, a_shape).astype(dtype)
        self.hB = rng.uniform(-1, 1, b_shape).astype(dtype)
        self.A = ng.array(self.hA, dtype=dtype)
        self.B = ng.array(self.hB, dtype=dtype)
        self.C = ng.empty(bshape + (m, n), dtype=dtype)
        self.C.rounding = 10 if sr else 0
        self.Aop = self.A.T if op[0] == "t" else self.A
        self.Bop = self.B.T if op[1] == "t" else self.B
        self.ng = ng
        self.flops = 2.0 * m * n * k * max(batch, 1)
        es = np.dtype(dtype).itemsize
        self.bytes = es * (m * k + k * n + m * n) * max(batch, 1)

    def name(self):
        return "%s%s %s m,n,k=%d,%d,%d%s%s" % ("batched%d " % self.batch if self.batch else "",
                                                np.dtype(self.dtype).name, self.op, self.m, self.n, self.k,
                                                " relu" if self.relu else "", " SR" if self.sr else "")

    def run(self):
        if self.batch:
            self.ng.batched_dot(self.Aop, self.Bop, self.C, relu=self.relu)
        else:
            self.ng.dot(self.Aop, self.Bop, self.C, relu=self.relu)

    def cpu(self):
        a = self.hA.astype(np.float32)
        b = self.hB.astype(np.float32)
        a = np.swapaxes(a, -1, -2) if self.op[0] == "t" else a
        b = np.swapaxes(b, -1, -2) if self.op[1] == "t" else b
        import oracle as orc
        if self.batch:
            return orc.ref_batched_dot(a, b, relu=self.relu, acc_dtype=np.float32)
        return orc.ref_dot(a, b, relu=self.relu, acc_dtype=np.float32)


SETTLE_MS = float(os.environ.get("NG_BENCH_SETTLE_MS", "60"))


def time_gpu(ng, fn, iters=20, warmup=3, settle_ms=None):
    """average duration in ms of fn() measured with HIP events on the launch stream.
    After an idle spell (the host preparing a case) the chip takes tens of
    milliseconds of work to reach its sustained clocks: the same kernel measured
    eight times in a row runs up to 18 % faster in the last measurement than in
    the first.  The untimed part therefore lasts at least `settle_ms` of GPU time
    (a pilot of `warmup` launches sizes it), so that what is timed is the
    sustained rate."""
    from nervanagpu_amd import _lib
    settle_ms = SETTLE_MS if settle_ms is None else settle_ms
    start, end = _lib.Event(), _lib.Event()
    warmup = max(warmup, 1)
    start.record(ng.stream)
    for _ in range(warmup):
        fn()
    end.record(ng.stream)
    end.synchronize()
    pilot = max(end.time_since(start) / warmup, 1e-3)
    for _ in range(min(int(settle_ms / pilot), 20000)):
        fn()
    start.record(ng.stream)
    for _ in range(iters):
        fn()
    end.record(ng.stream)
    end.synchronize()
    return end.time_since(start) / iters


LLC_BYTES = 256e6            # Infinity Cache of the MI355X: buffers cycled through must exceed it
COLD_BYTES = 640e6           # total footprint the rotating buffer sets of a "cold" row reach at least


def cold_sets(set_bytes):
    """number of buffer sets to rotate over so that a launch never finds its
    operands in the last-level cache: at least 3 sets and COLD_BYTES in total"""
    return int(max(3, -(-COLD_BYTES // max(set_bytes, 1))))


def time_gpu_rotating(ng, fns, iters=20, warmup=3):
    """like time_gpu, but launch k runs fns[k % len(fns)]: every fns[i] works on
    its own buffers, so consecutive launches do not re-read cached operands"""
    n = len(fns)
    count = -(-iters // n) * n
    state = {"i": 0}

    def one():
        fns[state["i"] % n]()
        state["i"] += 1
    return time_gpu(ng, one, count, max(warmup, n))


def build_config2(ng):
    cases = []
    for (M, K) in FC_SHAPES:
        for op in ("nn", "nt", "tn"):
            m, n, k = fc_mnk(op, M, K)
            for relu in (False, True):
                for sr in (False, True):
                    cases.append(GemmCase(ng, op, m, n, k, relu, sr))
    cases.append(GemmCase(ng, "nn", 4096, 4096, 4096))
    cases.append(GemmCase(ng, "nn", 512, 512, 512, batch=32))
    return cases


def blas_threads():
    try:
        from threadpoolctl import threadpool_info
        infos = [i for i in threadpool_info() if i.get("user_api") == "blas"]
        if infos:
            return int(infos[0]["num_threads"])
    except Exception:
        pass
    return int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))


CPU_BASELINE_SECONDS = 12.0


def cpu_baseline(cases):
    """np.dot oracle on a bounded sample of the step: repeated passes over the
    three FC nn shapes plus the 4096^3 case for about CPU_BASELINE_SECONDS of
    CPU work; the rate is total flops / total time"""
    sample = [c for c in cases if c.op == "nn" and not c.relu and not c.sr and not c.batch]
    flops = sum(c.flops for c in sample)
    for c in sample:
        c.cpu()                      # untimed first touch (BLAS thread pool, conversions)
    passes, t0 = 0, time.perf_counter()
    while True:
        for c in sample:
            c.cpu()
        passes += 1
        elapsed = time.perf_counter() - t0
        if elapsed >= CPU_BASELINE_SECONDS:
            break
    return {"value": flops * passes / elapsed / 1e12, "unit": "TFLOP/s", "cores": blas_threads(), "kind": "port",
            "sample": "np.dot (fp32 BLAS) over %s + 4096^3 nn, %d passes in %.1f s"
                      % (", ".join("(%d,%d)x128" % sh for sh in FC_SHAPES), passes, elapsed),
            "host_cpus": len(os.sched_getaffinity(0))}


# ---------------------------------------------------------------------------
# --all: every configured case with its own roofline
# ---------------------------------------------------------------------------

def cpu_seconds(fn, repeats=2):
    """best wall time of the oracle call fn() after one untimed first touch"""
    fn()
    best = None
    for _ in range(repeats):
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    return best


CPU_SAMPLE_PIXELS = 48      # output pixels per convolution layer timed on the CPU
CPU_SAMPLE_WINDOWS = 2048   # pooling windows timed on the CPU

ALEXNET = [(3, 224, 224, 64, 11, 11, 4, 2), (64, 27, 27, 192, 5, 5, 1, 2), (192, 13, 13, 384, 3, 3, 1, 1),
           (384, 13, 13, 256, 3, 3, 1, 1), (256, 13, 13, 256, 3, 3, 1, 1)]
VGG = [(3, 224, 64), (64, 224, 64), (64, 112, 128), (128, 112, 128), (128, 56, 256), (256, 56, 256),
       (256, 28, 512), (512, 28, 512), (512, 14, 512)]


def row(name, ms, flops=None, nbytes=None, peak_tflops=PEAK_FP16_TFLOPS, cpu=None, cache="warm", ms_warm=None):
    """One line of the per-case table.  `frac` is the fraction of the roofline that
    bounds the case: min(matrix peak, arithmetic intensity x HBM peak) for the
    contractions, HBM peak for pooling / elementwise.  cache: "cold" = timed over
    rotating buffer sets larger than the last-level cache (then ms_warm is the
    same case on one buffer set), "warm" = one buffer set re-used.
    cpu: (rate, unit, sample) of the numpy oracle on the host for the same case"""
    r = {"case": name, "ms": ms, "cache": cache}
    if ms_warm is not None:
        r["ms_warm"] = ms_warm
    if cpu:
        r["cpu_rate"], r["cpu_unit"], r["cpu_sample"] = cpu
    if flops:
        tf = flops / ms / 1e9
        r["tflops"] = tf
        r["pct_mfma_peak"] = 100.0 * tf / peak_tflops
        ceiling = peak_tflops
        if nbytes:
            ceiling = min(peak_tflops, flops / nbytes * PEAK_HBM_GBS / 1e3)
            r["pct_of_min_roof"] = 100.0 * tf / ceiling
        r["bound"] = "mfma" if ceiling >= peak_tflops else "hbm"
        r["frac"] = tf / ceiling
    if nbytes:
        r["gbs"] = nbytes / ms / 1e6
        if not flops:
            r["pct_hbm_peak"] = 100.0 * r["gbs"] / PEAK_HBM_GBS
            r["bound"] = "hbm"
            r["frac"] = r["gbs"] / PEAK_HBM_GBS
    return r


def hbm_bound(flops, nbytes, peak_tflops=PEAK_FP16_TFLOPS):
    return flops / nbytes * PEAK_HBM_GBS / 1e3 < peak_tflops


def conv_cpu(layer, rng):
    """the oracle's per-pixel gather + np.dot on a random sample of output pixels,
    scaled to the layer: (TFLOP/s, unit, sample)"""
    import oracle as orc
    M, P, Q = layer.MPQ
    I = np.full(layer.dimI, 0.5, dtype=np.float16)
    F = rng.standard_normal(layer.dimF).astype(np.float16)
    pixels = [(int(rng.integers(M)), int(rng.integers(P)), int(rng.integers(Q))) for _ in range(CPU_SAMPLE_PIXELS)]
    sec = cpu_seconds(lambda: orc.ref_conv_fprop_pixels(I, F, pixels, layer.padding, layer.strides, relu=True,
                                                        acc_dtype=np.float32), repeats=1)
    flops = layer.flops * len(pixels) / float(M * P * Q)
    return (flops / sec / 1e12, "TFLOP/s", "%d of %d output pixels" % (len(pixels), M * P * Q))


def conv_rows(ng, tag, N, layers, rows, iters, cpu=False):
    rng = np.random.default_rng(2)
    for cfg in layers:
        if tag == "conv3d":
            C, D, H, W, K, T, R, S = cfg
            layer = ng.conv_layer(np.float16, N, C, K, D, H, W, T, R, S)
        elif len(cfg) == 8:
            C, H, W, K, R, S, strd, pad = cfg
            layer = ng.conv_layer(np.float16, N, C, K, 1, H, W, 1, R, S, 0, pad, pad, 1, strd, strd)
        else:
            C, HW, K = cfg
            layer = ng.conv_layer(np.float16, N, C, K, 1, HW, HW, 1, 3, 3, 0, 1, 1, 1, 1, 1)
        sI, sF, sO = layer.sizeI * 2, layer.sizeF * 2, layer.sizeO * 2
        # layers priced by HBM (first layers, VGG conv1.2) are timed cold
        cold = hbm_bound(layer.flops, sI + sF + sO)
        nsets = cold_sets(sI + sO) if cold else 1
        sets = []
        for _ in range(nsets):
            I, F, E = ng.empty(layer.dimI), ng.empty(layer.dimF), ng.empty(layer.dimO)
            O, B, U = ng.empty(layer.dimO), ng.empty(layer.dimI), ng.empty(layer.dimF, dtype=np.float32)
            I[:] = ng.rand()
            E[:] = ng.rand() - 0.5
            F[:] = (ng.rand() - 0.5) * 0.05
            sets.append((I, F, E, O, B, U))
        nm = "%s C%d K%d %s %s" % (tag, layer.C, layer.K, layer.DHW, layer.TRS)
        ops = [("fprop", lambda t: ng.fprop_conv(layer, t[0], t[1], t[3], relu=True), sI + sF + sO)]
        if tag != "conv3d":
            ops.append(("bprop", lambda t: ng.bprop_conv(layer, t[1], t[2], t[4]), sI + sF + sO))
            ops.append(("update", lambda t: ng.update_conv(layer, t[0], t[2], t[5]), sI + sO + layer.sizeF * 4))
        for opname, fn, nbytes in ops:
            warm = time_gpu(ng, lambda: fn(sets[0]), iters)
            ms = time_gpu_rotating(ng, [(lambda t=t: fn(t)) for t in sets], iters) if cold else warm
            rows.append(row("%s %s" % (nm, opname), ms, layer.flops, nbytes, cache="cold" if cold else "warm",
                            ms_warm=warm if cold else None,
                            cpu=conv_cpu(layer, rng) if (cpu and opname == "fprop") else None))
        del sets


def pool_cpu(layer, nbytes):
    """the oracle's gather + np.max / np.mean on a random sample of windows,
    scaled to the layer's algorithmic bytes: (GB/s, unit, sample)"""
    import oracle as orc
    rng = np.random.default_rng(3)
    K, M, P, Q = layer.K, layer.MPQ[0], layer.MPQ[1], layer.MPQ[2]
    I = np.full(layer.dimI, 0.5, dtype=np.float16)
    windows = [(int(rng.integers(K)), int(rng.integers(M)), int(rng.integers(P)), int(rng.integers(Q)))
               for _ in range(CPU_SAMPLE_WINDOWS)]
    sec = cpu_seconds(lambda: orc.ref_pool_fprop_pixels(I, layer.op, layer.JTRS, windows, layer.padding, layer.strides),
                      repeats=1)
    total = K * M * P * Q
    return (nbytes * len(windows) / float(total) / sec / 1e9, "GB/s", "%d of %d windows" % (len(windows), total))


def pool_rows(ng, tag, N, C, HW, win, strd, op, rows, iters, cpu=False):
    layer = ng.pool_layer(np.float16, op, N, C, 1, HW, HW, 1, 1, win, win, 0, 0, 0, 0, 1, 1, strd, strd)
    sI, sO = layer.sizeI * 2, layer.sizeO * 2
    sets = []
    for _ in range(cold_sets(2 * sI + 2 * sO)):
        I, E, O, B = ng.empty(layer.dimI), ng.empty(layer.dimO), ng.empty(layer.dimO), ng.empty(layer.dimI)
        I[:] = ng.rand()
        E[:] = ng.rand()
        sets.append((I, E, O, B))
    nm = "%s %s %dx%d/%d C%d %dx%d N%d" % (tag, op, win, win, strd, C, HW, HW, N)
    warm = time_gpu(ng, lambda: ng.fprop_pool(layer, sets[0][0], sets[0][2]), iters)
    ms = time_gpu_rotating(ng, [(lambda t=t: ng.fprop_pool(layer, t[0], t[2])) for t in sets], iters)
    rows.append(row(nm + " fprop", ms, None, sI + sO, cache="cold", ms_warm=warm,
                    cpu=pool_cpu(layer, sI + sO) if cpu else None))
    warm = time_gpu(ng, lambda: ng.bprop_pool(layer, sets[0][0], sets[0][1], sets[0][3]), iters)
    ms = time_gpu_rotating(ng, [(lambda t=t: ng.bprop_pool(layer, t[0], t[1], t[3])) for t in sets], iters)
    rows.append(row(nm + " bprop", ms, None, (2 * sI + sO) if op == "max" else (sI + sO), cache="cold", ms_warm=warm))


def gemm_row(ng, prefix, c, iters, peak=PEAK_FP16_TFLOPS, cpu=None):
    """GEMM shapes priced by HBM (minibatch-wide, batched) are timed cold: the
    same product over rotating operand sets; matrix-bound shapes on one set"""
    if not hbm_bound(c.flops, c.bytes, peak):
        return row(prefix + c.name(), time_gpu(ng, c.run, iters), c.flops, c.bytes, peak, cpu=cpu)
    clones = [c] + [GemmCase(ng, c.op, c.m, c.n, c.k, c.relu, c.sr, c.dtype, c.batch, seed=100 + i)
                    for i in range(cold_sets(c.bytes) - 1)]
    warm = time_gpu(ng, c.run, iters)
    ms = time_gpu_rotating(ng, [x.run for x in clones], iters)
    return row(prefix + c.name(), ms, c.flops, c.bytes, peak, cpu=cpu, cache="cold", ms_warm=warm)


def all_cases(ng, cases, iters=10, cpu=False):
    """Every configured case of configs 1-5 with its own roofline fraction.
    cpu: also time the numpy oracle on the host for one case of every kind
    (np.dot for the GEMMs, sampled pixels / windows for convolution and pooling
    forward, the whole array for the elementwise cases)"""
    from nervanagpu_amd import NervanaGPU
    import oracle as orc
    rows = []

    def gemm_cpu(c):
        if not cpu:
            return None
        return (c.flops / cpu_seconds(c.cpu, repeats=1) / 1e12, "TFLOP/s", "np.dot, fp32 BLAS, %d threads" % blas_threads())
    # config 1
    for op in ("nn", "tn"):
        c = GemmCase(ng, op, 1024, 1024, 1024, dtype=np.float32, seed=0)
        rows.append(gemm_row(ng, "cfg1 ", c, iters, PEAK_FP32_TFLOPS, gemm_cpu(c)))
    # config 2
    for c in cases:
        if c.relu or c.sr:
            continue
        rows.append(gemm_row(ng, "cfg2 ", c, iters, cpu=gemm_cpu(c) if c.op == "nn" else None))
    for op in ("nt", "tn"):
        rows.append(gemm_row(ng, "cfg2 ", GemmCase(ng, op, 4096, 4096, 4096), iters))
    for c in cases:
        if c.sr and c.relu and c.op == "nn":
            rows.append(gemm_row(ng, "cfg2 ", c, iters))
    conv_rows(ng, "cfg3 alexnet", 128, ALEXNET, rows, iters, cpu)
    conv_rows(ng, "cfg4 vgg", 64, VGG, rows, iters, cpu)
    for (C, HW) in ((64, 224), (128, 112), (256, 56), (512, 28), (512, 14)):
        pool_rows(ng, "cfg4", 64, C, HW, 2, 2, "max", rows, iters, cpu and HW == 224)
    # config 5
    ngs = NervanaGPU(stochastic_round=True, seed=4)
    nsets = cold_sets(2 * 4096 * 8192 * 2)
    As = [ngs.empty((4096, 8192)) for _ in range(nsets)]
    Bs = [ngs.empty((4096, 8192)) for _ in range(nsets)]
    for A in As:
        A[:] = ngs.rand()

    def bn(A):
        A[:] = (A - ngs.mean(A, axis=1)) / ngs.sqrt(ngs.var(A, axis=1) + 1e-3)
    hA = np.random.default_rng(4).uniform(0, 1, (4096, 8192)).astype(np.float16) if cpu else None
    bn_cpu = ew_cpu = None
    if cpu:
        sec = cpu_seconds(lambda: orc.ref_batchnorm_rows(hA, 1e-3).astype(np.float16), repeats=1)
        bn_cpu = (2 * hA.nbytes / sec / 1e9, "GB/s", "numpy, whole array")
        h32 = hA.astype(np.float32)
        sec = cpu_seconds(lambda: (h32 * h32 + h32).astype(np.float16), repeats=1)
        ew_cpu = (2 * hA.nbytes / sec / 1e9, "GB/s", "numpy, whole array")
    nb = 2 * As[0].nbytes
    rows.append(row("cfg5 batchnorm (4096,8192) fp16 SR", time_gpu_rotating(ngs, [(lambda A=A: bn(A)) for A in As], iters),
                    None, nb, cpu=bn_cpu, cache="cold", ms_warm=time_gpu(ngs, lambda: bn(As[0]), iters)))
    for B in Bs:
        B.rounding = 0
    rows.append(row("cfg5 batchnorm (4096,8192) fp16 nearest",
                    time_gpu_rotating(ngs, [(lambda A=A, B=B: B._assign((A - ngs.mean(A, axis=1)) / ngs.sqrt(ngs.var(A, axis=1) + 1e-3)))
                                            for A, B in zip(As, Bs)], iters), None, nb, cache="cold"))
    rows.append(row("cfg5 elementwise a*a+a (4096,8192) fp16",
                    time_gpu_rotating(ngs, [(lambda A=A, B=B: B._assign(A * A + A)) for A, B in zip(As, Bs)], iters),
                    None, nb, cpu=ew_cpu, cache="cold", ms_warm=time_gpu(ngs, lambda: Bs[0]._assign(As[0] * As[0] + As[0]), iters)))
    # yardstick for the bandwidth rows: a plain device-to-device copy of the same
    # footprint (64 MiB in, 64 MiB out), through the same rotation
    rows.append(row("cfg5 plain copy (4096,8192) fp16 [yardstick]",
                    time_gpu_rotating(ngs, [(lambda A=A, B=B: B._assign(A)) for A, B in zip(As, Bs)], iters),
                    None, nb, cache="cold", ms_warm=time_gpu(ngs, lambda: Bs[0]._assign(As[0]), iters)))
    del As, Bs
    for op in ("max", "avg"):
        pool_rows(ng, "cfg5", 128, 256, 56, 3, 2, op, rows, iters, cpu)
    conv_rows(ng, "conv3d", 32, [(64, 16, 28, 28, 128, 3, 3, 3)], rows, iters, cpu)
    return rows


def format_rows(rows):
    lines = ["| case | GPU ms | cache | ms warm | TFLOP/s | % MFMA peak | % of min(MFMA, AI*BW) | GB/s | % HBM peak | CPU oracle |",
             "|---|---|---|---|---|---|---|---|---|---|"]
    for r in rows:
        lines.append("| %s | %.4f | %s | %s | %s | %s | %s | %s | %s | %s |" % (
            r["case"], r["ms"], r.get("cache", ""),
            "%.4f" % r["ms_warm"] if "ms_warm" in r else "",
            "%.1f" % r["tflops"] if "tflops" in r else "",
            "%.1f" % r["pct_mfma_peak"] if "pct_mfma_peak" in r else "",
            "%.1f" % r["pct_of_min_roof"] if "pct_of_min_roof" in r else "",
            "%.0f" % r["gbs"] if "gbs" in r else "",
            "%.1f" % r["pct_hbm_peak"] if "pct_hbm_peak" in r else "",
            "%.3g %s (%s)" % (r["cpu_rate"], r["cpu_unit"], r["cpu_sample"]) if "cpu_rate" in r else ""))
    return "\n".join(lines)


def compact(rows):
    """the per-case rows as they go into the JSON line: short keys, rounded"""
    out = []
    for r in rows:
        c = {"case": r["case"], "ms": round(r["ms"], 5), "cache": r["cache"], "bound": r["bound"], "frac": round(r["frac"], 4)}
        if "ms_warm" in r:
            c["ms_warm"] = round(r["ms_warm"], 5)
        if "tflops" in r:
            c["tflops"] = round(r["tflops"], 1)
        else:
            c["gbs"] = round(r["gbs"], 0)
        if "cpu_rate" in r:
            c["cpu"] = "%.3g %s (%s)" % (r["cpu_rate"], r["cpu_unit"], r["cpu_sample"])
        out.append(c)
    return out


TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemm_4096_fp16_hbm_traffic.md")


def dominant_traffic():
    """HBM bytes per launch of the 4096^3 kernel as measured with rocprofv3 --pmc
    FETCH_SIZE / WRITE_SIZE on `bench.py --calibrate` (each counter scaled by its
    reading for the 256 MiB copy of the same run); the committed summary of that
    measurement carries the figure on a line `traffic_bytes_per_launch: N`.
    Counters cannot be read from inside this process, so the line is the source."""
    try:
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return float(line.split(":", 1)[1].split()[0])
    except OSError:
        pass
    return None


CAL_COPY_ELEMS = 1 << 27     # fp16 elements of the calibration copy: 256 MiB read + 256 MiB written


def profile_cases(ng):
    """name -> (description, callable) of the single launches hardware counters are collected on"""
    from nervanagpu_amd import NervanaGPU
    out = {}

    def gemm(op):
        c = GemmCase(ng, op, 4096, 4096, 4096)
        return (c.name(), c.run)
    out["gemm"] = lambda: gemm("nn")
    out["gemm_nt"] = lambda: gemm("nt")

    def fc():
        c = GemmCase(ng, "nn", 4096, 128, 9216)
        return (c.name(), c.run)
    out["fc"] = fc

    def conv(C, HW, K, which):
        layer = ng.conv_layer(np.float16, 64, C, K, 1, HW, HW, 1, 3, 3, 0, 1, 1, 1, 1, 1)
        I, F, E = ng.empty(layer.dimI), ng.empty(layer.dimF), ng.empty(layer.dimO)
        O, B, U = ng.empty(layer.dimO), ng.empty(layer.dimI), ng.empty(layer.dimF, dtype=np.float32)
        I[:] = ng.rand()
        E[:] = ng.rand() - 0.5
        F[:] = (ng.rand() - 0.5) * 0.05
        fn = {"fprop": lambda: ng.fprop_conv(layer, I, F, O, relu=True),
              "bprop": lambda: ng.bprop_conv(layer, F, E, B),
              "update": lambda: ng.update_conv(layer, I, E, U)}[which]
        return ("vgg conv C%d K%d %dx%d N64 %s: I %d B, F %d B, O %d B" % (C, K, HW, HW, which, layer.sizeI * 2,
                                                                          layer.sizeF * 2, layer.sizeO * 2), fn)
    for which in ("fprop", "bprop", "update"):
        out["conv64_" + which] = lambda which=which: conv(64, 224, 64, which)
        out["conv512_" + which] = lambda which=which: conv(512, 28, 512, which)
        out["conv3_" + which] = lambda which=which: conv(3, 224, 64, which)

    def pool(which):
        layer = ng.pool_layer(np.float16, "max", 128, 256, 1, 56, 56, 1, 1, 3, 3, 0, 0, 0, 0, 1, 1, 2, 2)
        I, E, O, B = ng.empty(layer.dimI), ng.empty(layer.dimO), ng.empty(layer.dimO), ng.empty(layer.dimI)
        I[:] = ng.rand()
        E[:] = ng.rand()
        fn = (lambda: ng.fprop_pool(layer, I, O)) if which == "fprop" else (lambda: ng.bprop_pool(layer, I, E, B))
        return ("max pool 3x3/2 C256 56x56 N128 %s: I %d B, O %d B" % (which, layer.sizeI * 2, layer.sizeO * 2), fn)
    out["pool_fprop"] = lambda: pool("fprop")
    out["pool_bprop"] = lambda: pool("bprop")

    def bn():
        ngs = NervanaGPU(stochastic_round=True, seed=4)
        A = ngs.empty((4096, 8192))
        A[:] = ngs.rand()

        def run():
            A[:] = (A - ngs.mean(A, axis=1)) / ngs.sqrt(ngs.var(A, axis=1) + 1e-3)
        return ("batch normalisation (4096,8192) fp16 in place, stochastic store: %d B read, %d B written" % (A.nbytes, A.nbytes), run)
    out["bn"] = bn
    return out


def calibrate(ng, names):
    """Counter collection run: a flat copy kernel that reads and writes exactly
    CAL_COPY_ELEMS * 2 bytes, then each named case, five launches each."""
    from nervanagpu_amd import _lib
    src = ng.empty((CAL_COPY_ELEMS // 8192, 8192), dtype=np.float16)
    dst = ng.empty((CAL_COPY_ELEMS // 8192, 8192), dtype=np.float16)
    src.fill(1.0)
    for _ in range(5):
        dst._assign(src)
    table = profile_cases(ng)
    done = {}
    for name in names:
        if name not in table:
            sys.exit("bench.py --calibrate: unknown case %r (known: %s)" % (name, ", ".join(sorted(table))))
        desc, fn = table[name]()
        for _ in range(5):
            fn()
        _lib.stream_sync(ng.stream)
        done[name] = desc
    print(json.dumps({"calibrate": {"copy_bytes_read": CAL_COPY_ELEMS * 2, "copy_bytes_written": CAL_COPY_ELEMS * 2,
                                    "cases": done}}))


MFMA_LOOP_SOURCE = r"""
typedef _Float16 half8_t   __attribute__((ext_vector_type(8)));
typedef float    float16_t __attribute__((ext_vector_type(16)));

// 256 threads = one wavefront per SIMD; 16 independent 32x32 accumulators per
// wavefront, so the matrix pipe never waits on a dependency; no memory traffic
extern "C" __global__ __launch_bounds__(256)
void mfma_loop(float* out, int iters, int random_data)
{
    half8_t a, b;
    unsigned h = (blockIdx.x * 256u + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        h ^= h >> 15; h *= 0x2c1b3c6du; h ^= h >> 12; h *= 0x297a2d39u; h ^= h >> 15;
        a[i] = random_data ? (_Float16)(((int)(h & 2047) - 1024) * (1.0f / 1024)) : (_Float16)1.0f;
        b[i] = random_data ? (_Float16)(((int)((h >> 11) & 2047) - 1024) * (1.0f / 1024)) : (_Float16)0.5f;
    }
    float16_t acc[16];
#pragma unroll
    for (int j = 0; j < 16; j++)
#pragma unroll
        for (int v = 0; v < 16; v++) acc[j][v] = 0.0f;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int j = 0; j < 16; j++) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[j], 0, 0, 0);
    }
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 16; j++)
#pragma unroll
        for (int v = 0; v < 16; v++) s += acc[j][v];
    out[blockIdx.x * 256u + threadIdx.x] = s;
}
"""


def mfma_ceiling(ng):
    """A loop of back-to-back MFMAs without memory traffic (compiled at run time
    from MFMA_LOOP_SOURCE; a yardstick, not part of the library), two workgroups
    of four wavefronts per CU, on constant and on random operands: what the
    matrix pipes deliver at the clock the power limit allows."""
    import ctypes
    from nervanagpu_amd import _lib
    blocks, out = 512, {}
    buf = ng.empty((blocks, 256), dtype=np.float32)
    kernel = _lib.Module(MFMA_LOOP_SOURCE, "mfma_loop").get_function("mfma_loop")
    for label, rnd in (("constant", 0), ("random", 1)):
        for iters in (4000, 40000):
            def run():
                kernel.launch((blocks, 1, 1), (256, 1, 1), ng.stream,
                              [ctypes.c_void_p(buf.ptr), ctypes.c_int(iters), ctypes.c_int(rnd)])
            ms = time_gpu(ng, run, iters=5, warmup=1)
            out["%s operands, %d rounds (%.2f ms)" % (label, iters, ms)] = blocks * 4 * iters * 16 * 32768.0 / ms / 1e9
    print(json.dumps({"mfma_ceiling_tflops": out, "peak": PEAK_FP16_TFLOPS}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=60,
                    help="untimed steps (a step is about 1 ms; the chip needs tens of ms to reach its sustained clocks)")
    ap.add_argument("--all", action="store_true", help="print the per-case table (stderr, or --out FILE)")
    ap.add_argument("--out", default=None, help="file for the per-case table")
    ap.add_argument("--no-cases", action="store_true", help="only the headline step, no per-case rows")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calibrate", nargs="?", const="gemm", default=None, metavar="CASES",
                    help="only launch a plain copy of known size and the named cases (comma separated; "
                         "default the dominant GEMM) five times each: the run hardware counters are collected on")
    ap.add_argument("--mfma-ceiling", action="store_true",
                    help="only time the MFMA loop without memory traffic (practical matrix-pipe ceiling)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (got --gpus %d); "
                 "the data-parallel path has no collective step on one device" % args.gpus)

    from nervanagpu_amd import NervanaGPU, _lib
    ng = NervanaGPU(stochastic_round=False, bench=False, seed=1)
    if args.calibrate:
        calibrate(ng, [n for n in args.calibrate.split(",") if n])
        return
    if args.mfma_ceiling:
        mfma_ceiling(ng)
        return
    cases = build_config2(ng)
    step_flops = sum(c.flops for c in cases)

    def step():
        for c in cases:
            c.run()

    for _ in range(args.warmup):
        step()
    _lib.stream_sync(ng.stream)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    _lib.stream_sync(ng.stream)
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps

    dominant = [c for c in cases if c.m == c.n == c.k == 4096][0]
    dom_ms = time_gpu(ng, dominant.run, iters=max(args.steps, 20), warmup=3)
    achieved = dominant.flops / dom_ms / 1e9
    roofline = {"bound": "mfma", "kernel": "mfma_gemm_direct_kernel<fp16,256x256x64,A:KC,B:MC,2 stages> (4096^3 nn)",
                "achieved": achieved, "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                "frac": achieved / PEAK_FP16_TFLOPS, "traffic": dominant_traffic(),
                "traffic_source": "profiles/gemm_4096_fp16_hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE; "
                                  "not re-measured by this run)",
                "launch_ms": dom_ms, "flops_per_launch": dominant.flops}

    result = {
        "metric": "fp16 GEMM/conv TFLOP/s + % MFMA peak; pool/elementwise GB/s on 1 MI355X",
        "value": step_flops / (ms_per_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "config 2: fp16 FC GEMM sweep N=128 (3 shapes x nn/nt/tn x relu x RN/SR) "
                               "+ 4096^3 nn + batched 32x512^3; %d GEMM launches per step" % len(cases),
                   "flops_per_step": step_flops},
        "roofline": roofline,
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(cases)

    if not args.no_cases:
        # one row per kernel family and configured shape, timed in this same run:
        # GEMM (configs 1, 2), convolution fprop/bprop/update (3, 4, 3-D), pooling,
        # batch normalisation and elementwise (5); HBM-priced rows over rotating buffers
        rows = all_cases(ng, cases, cpu=not args.no_cpu)
        if args.all or args.out:
            table = format_rows(rows)
            if args.out:
                with open(args.out, "w") as f:
                    f.write(table + "\n")
            else:
                sys.stderr.write(table + "\n")
        result["cases"] = compact(rows)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
