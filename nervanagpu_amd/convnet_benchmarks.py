#!/usr/bin/env python3
"""
Whole-network forward / backward timing of the classic convnets, the way the
reference measures them (benchmarks/convnet-benchmarks.py:120-200, 250-403):
layers are created with Layer.create, activations per layer, two alternating
shared delta buffers and one shared fp32 update buffer, initial weights scaled by
a first forward pass so activations stay near 1, then `loops` timed iterations
of fprop over all layers and bprop (data gradient + weight gradient) from the
last layer back to the first.

    python -m nervanagpu_amd.convnet_benchmarks [--nets Alexnet,VGG] [--dtypes f16,f32]
                                                [--loops 10] [--json FILE] [--zeros]

"gflops" counts the multiply-adds of the conv and fully connected layers only
and bprop as twice fprop, as the reference does (nervanagpu/layers.py:243,422;
benchmarks/convnet-benchmarks.py:375).  The published figures of the reference
(README.md:140-187, one GTX Titan X) are printed beside the measured ones.
"""
import argparse
import json
import sys
from functools import reduce
from operator import mul

import numpy as np

from . import NervanaGPU, _lib
from .layers import Layer, DataLayer, ConvLayer, PoolLayer, FullLayer, Inception

# layer shorthands: ("conv", K, R, pad, stride) / ("pool", R, stride[, pad[, op]]) / ("full", nOut)
# ("incep1", widths) / ("incep2", widths): the two inception module shapes, see _inception()
_STEM = [("conv", 64, 7, 3, 2), ("pool", 3, 2, 1), ("conv", 64, 1, 0, 1), ("conv", 192, 3, 1, 1), ("pool", 3, 2, 1)]
_NETS = {
    "Alexnet": dict(N=128, H=224, warmup=5, layers=[
        ("conv", 64, 11, 2, 4), ("pool", 3, 2), ("conv", 192, 5, 2, 1), ("pool", 3, 2),
        ("conv", 384, 3, 1, 1), ("conv", 256, 3, 1, 1), ("conv", 256, 3, 1, 1), ("pool", 3, 2),
        ("full", 3072), ("full", 3072), ("full", 1000)]),
    "Overfeat": dict(N=128, H=231, warmup=1, layers=[
        ("conv", 96, 11, 0, 4), ("pool", 2, 2), ("conv", 256, 5, 0, 1), ("pool", 2, 2),
        ("conv", 512, 3, 1, 1), ("conv", 1024, 3, 1, 1), ("conv", 1024, 3, 1, 1), ("pool", 2, 2),
        ("full", 3072), ("full", 3072), ("full", 1000)]),
    "VGG": dict(N=64, H=224, warmup=1, layers=[
        ("conv", 64, 3, 1, 1), ("pool", 2, 2), ("conv", 128, 3, 1, 1), ("pool", 2, 2),
        ("conv", 256, 3, 1, 1), ("conv", 256, 3, 1, 1), ("pool", 2, 2),
        ("conv", 512, 3, 1, 1), ("conv", 512, 3, 1, 1), ("pool", 2, 2),
        ("conv", 512, 3, 1, 1), ("conv", 512, 3, 1, 1), ("pool", 2, 2),
        ("full", 3072), ("full", 3072), ("full", 1000)]),
    "VGG_E": dict(N=64, H=224, warmup=1, layers=[
        ("conv", 64, 3, 1, 1), ("conv", 64, 3, 1, 1), ("pool", 2, 2),
        ("conv", 128, 3, 1, 1), ("conv", 128, 3, 1, 1), ("pool", 2, 2)] +
        [("conv", 256, 3, 1, 1)] * 4 + [("pool", 2, 2)] +
        [("conv", 512, 3, 1, 1)] * 4 + [("pool", 2, 2)] +
        [("conv", 512, 3, 1, 1)] * 4 + [("pool", 2, 2)] +
        [("full", 3072), ("full", 3072), ("full", 1000)]),
    # http://arxiv.org/abs/1409.4842
    "GoogLeNet1": dict(N=128, H=224, warmup=1, layers=_STEM + [
        ("incep1", ((64,), (96, 128), (16, 32), (32,))),
        ("incep1", ((128,), (128, 192), (32, 96), (64,))), ("pool", 3, 2, 1),
        ("incep1", ((192,), (96, 208), (16, 48), (64,))),
        ("incep1", ((160,), (112, 224), (24, 64), (64,))),
        ("incep1", ((128,), (128, 256), (24, 64), (64,))),
        ("incep1", ((112,), (144, 288), (32, 64), (64,))),
        ("incep1", ((256,), (160, 320), (32, 128), (128,))), ("pool", 3, 2, 1),
        ("incep1", ((256,), (160, 320), (32, 128), (128,))),
        ("incep1", ((384,), (192, 384), (48, 128), (128,))),
        ("pool", 7, 1, 0, "avg"), ("full", 1000)]),
    # the batch-normalised variant's shapes (http://arxiv.org/abs/1502.03167), without the normalisation
    "GoogLeNet2": dict(N=128, H=224, warmup=1, layers=_STEM + [
        ("incep2", ((64,), (64, 64), (64, 96), ("avg", 32))),
        ("incep2", ((64,), (64, 96), (64, 96), ("avg", 64))),
        ("incep2", ((0,), (128, 160), (64, 96), ("max", 0))), ("conv", 576, 2, 0, 2),
        ("incep2", ((224,), (64, 96), (96, 128), ("avg", 128))),
        ("incep2", ((192,), (96, 128), (96, 128), ("avg", 128))),
        ("incep2", ((160,), (128, 160), (128, 160), ("avg", 96))),
        ("incep2", ((96,), (128, 192), (160, 192), ("avg", 96))),
        ("incep2", ((0,), (128, 192), (192, 256), ("max", 0))), ("conv", 1024, 2, 0, 2),
        ("incep2", ((352,), (192, 320), (160, 224), ("avg", 128))),
        ("incep2", ((352,), (192, 320), (192, 224), ("max", 128))),
        ("pool", 7, 1, 0, "avg"), ("full", 1000)]),
}

# reference README.md:140-187: (fprop ms, bprop ms, total ms) on one GTX Titan X
PUBLISHED_TITAN_X_MS = {
    ("Alexnet", "float16"): (28.341, 60.768, 89.109), ("Alexnet", "float32"): (29.332, 66.216, 95.548),
    ("Overfeat", "float16"): (107.401, 236.339, 343.741), ("Overfeat", "float32"): (117.611, 268.379, 385.990),
    ("VGG", "float16"): (153.939, 337.443, 491.382), ("VGG", "float32"): (165.948, 389.139, 555.087),
    ("VGG_E", "float16"): (396.107, 854.090, 1250.197), ("VGG_E", "float32"): (435.622, 971.928, 1407.550),
}


def _conv(K, R, pad=0, strd=1):
    return {"layer": ConvLayer, "K": K, "R": R, "S": R, "pad_h": pad, "pad_w": pad, "str_h": strd, "str_w": strd}


def _pool(R, strd, pad=0, op="max"):
    return {"layer": PoolLayer, "op": op, "R": R, "S": R, "str_h": strd, "str_w": strd, "pad_h": pad, "pad_w": pad}


def _inception(kind, w):
    """Inception configuration from its branch widths (reference
    benchmarks/convnet-benchmarks.py:76-118).  "incep1": 1x1 | 1x1 -> 3x3 |
    1x1 -> 5x5 | 3x3 max pool -> 1x1.  "incep2": [1x1] | 1x1 -> 3x3 |
    1x1 -> 3x3 -> 3x3 | 3x3 pool (w[3][0] names the op) [-> 1x1]; a zero width
    drops the bracketed layer."""
    if kind == "incep1":
        parts = [(_conv(w[0][0], 1),),
                 (_conv(w[1][0], 1), _conv(w[1][1], 3, 1)),
                 (_conv(w[2][0], 1), _conv(w[2][1], 5, 2)),
                 (_pool(3, 1, 1), _conv(w[3][0], 1))]
    else:
        parts = [(_conv(w[0][0], 1),)] if w[0][0] else []
        parts += [(_conv(w[1][0], 1), _conv(w[1][1], 3, 1)),
                  (_conv(w[2][0], 1), _conv(w[2][1], 3, 1), _conv(w[2][1], 3, 1))]
        tail = (_pool(3, 1, 1, w[3][0]),)
        parts.append(tail + (_conv(w[3][1], 1),) if w[3][1] else tail)
    return {"layer": Inception, "partitions": tuple(parts)}


def network_config(name):
    """list of Layer.create configuration dicts for a named network"""
    net = _NETS[name]
    confs = [{"layer": DataLayer, "N": net["N"], "C": 3, "H": net["H"], "W": net["H"]}]
    for spec in net["layers"]:
        if spec[0] == "conv":
            confs.append(_conv(*spec[1:]))
        elif spec[0] == "pool":
            confs.append(_pool(*spec[1:]))
        elif spec[0] in ("incep1", "incep2"):
            confs.append(_inception(*spec))
        else:
            confs.append({"layer": FullLayer, "nOut": spec[1]})
    return confs


def fold_relu_derivatives(layers):
    """Let the backward kernel of the layer above apply a convolution or fully
    connected layer's rectifier derivative, so that layer skips its elementwise
    pass over the errors.  A max pooling layer above reads the same activations
    to find its maxima (no extra traffic); a unit-stride convolution above
    reads them once in its store.  Same results; not part of the reference's
    driver.  Returns the number of folded pairs."""
    folded = 0
    for below, above in zip(layers[:-1], layers[1:]):
        if type(below) not in (ConvLayer, FullLayer):
            continue
        if type(above) is PoolLayer and above.op == "max" and reduce(mul, above.JTRS, 1) <= 255:
            above.relu_below = True
        elif type(above) is ConvLayer and tuple(above.strides) == (1, 1, 1) and above.bprop_out is not None:
            above.relu_mask_below = below.fprop_out
        else:
            continue
        below.relu_done_above = True
        folded += 1
    return folded


def build_network(ng, confs, dtype, zeros=False, seed=0, fold_relu=False):
    """create the layers, their activations, the shared delta / update buffers and
    scaled initial weights; returns the layer list"""
    layers, prev = [], None
    max_deltas, max_weights = 0, 0
    max_delta_layer = max_weight_layer = None
    for conf in confs:
        layer = Layer.create(ng, conf, prev, dtype)
        if layer.sizeF > max_weights:
            max_weights, max_weight_layer = layer.sizeF, layer
        if layer.sizeI > max_deltas and type(prev) is not DataLayer:
            max_deltas, max_delta_layer = layer.sizeI, layer
        prev = layer
        layers.append(layer)

    # two alternating buffers: a layer cannot read and write its errors in one buffer;
    # the branches inside an inception layer alternate between two more
    nbuf = 4 if any(type(l) is Inception for l in layers) else 2
    shared_deltas = [ng.empty(max_delta_layer.dimI, dtype=max_delta_layer.dtype) for _ in range(nbuf)]
    shared_updates = ng.empty(max_weight_layer.dimF, dtype=np.float32)
    np.random.seed(seed)
    for i, layer in enumerate(layers):
        layer.init_activations()
        layer.init_weights(shared=shared_updates, zeros=zeros)
        if i > 1:
            layer.init_deltas(shared=shared_deltas)

    if zeros:
        layers[0].init_data()
    else:
        layers[0].init_data(np.random.uniform(0.0, 1.0, layers[0].dimO))
        # scale the initial weights so that activations stay bound around 1
        bench, ng.bench = ng.bench, False
        propagation = None
        for layer in layers:
            propagation = layer.fprop(propagation, scale_weights=.5)
        ng.bench = bench
    if fold_relu:
        fold_relu_derivatives(layers)
    return layers


def run_network(ng, name, dtype, loops=10, zeros=False, verbose=True, out=sys.stdout, fold_relu=False, warmup=None):
    net = _NETS[name]
    layers = build_network(ng, network_config(name), dtype, zeros=zeros, fold_relu=fold_relu)
    start, end = _lib.Event(), _lib.Event()
    # untimed iterations: the reference's count unless the caller asks for more (sustained clocks)
    warmup = net["warmup"] if warmup is None else max(int(warmup), net["warmup"])
    fprop_ms = bprop_ms = 0.0
    fprop_flops = bprop_flops = 0
    for loop in range(loops + warmup):
        count = max(loop - warmup + 1, 0)

        start.record(ng.stream)
        flops = 0
        propagation = None
        for layer in layers:
            propagation = layer.fprop(propagation)
            flops += layer.flops
        end.record(ng.stream)
        end.synchronize()
        msecs = end.time_since(start)
        if verbose:
            out.write("fprop(%2d): %8.3f msecs %8.3f gflops\n" % (count, msecs, flops / (msecs * 1e6)))
        if count > 0:
            fprop_ms += msecs
            fprop_flops += flops

        start.record(ng.stream)
        flops = 0
        for layer in layers[:0:-1]:
            propagation = layer.bprop(propagation)
            flops += layer.flops * 2
        end.record(ng.stream)
        end.synchronize()
        msecs = end.time_since(start)
        if verbose:
            out.write("bprop(%2d): %8.3f msecs %8.3f gflops\n" % (count, msecs, flops / (msecs * 1e6)))
        if count > 0:
            bprop_ms += msecs
            bprop_flops += flops

    res = {"net": name, "dtype": np.dtype(dtype).name, "N": net["N"], "loops": loops, "fold_relu": bool(fold_relu),
           "fprop_ms": fprop_ms / loops, "bprop_ms": bprop_ms / loops, "total_ms": (fprop_ms + bprop_ms) / loops,
           "fprop_gflops": fprop_flops / (fprop_ms * 1e6), "bprop_gflops": bprop_flops / (bprop_ms * 1e6),
           "total_gflops": (fprop_flops + bprop_flops) / ((fprop_ms + bprop_ms) * 1e6)}
    pub = PUBLISHED_TITAN_X_MS.get((name, res["dtype"]))
    if pub:
        res["published_titan_x_ms"] = {"fprop": pub[0], "bprop": pub[1], "total": pub[2]}
        res["speedup_vs_published_total"] = pub[2] / res["total_ms"]
    return res


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--nets", default="Alexnet,Overfeat,VGG,VGG_E")
    ap.add_argument("--dtypes", default="f16,f32")
    ap.add_argument("--loops", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed iterations before the timed ones (default: the reference's 1, Alexnet 5)")
    ap.add_argument("--zeros", action="store_true", help="all-zero data and weights")
    ap.add_argument("--quiet", action="store_true", help="only the per-network summary")
    ap.add_argument("--json", default=None, help="write the summaries to this file")
    ap.add_argument("--fold-relu", action="store_true",
                    help="let max pooling and unit-stride convolution backward apply the rectifier derivative of "
                         "the layer below them (same results, one elementwise pass per such pair saved; not in "
                         "the reference)")
    args = ap.parse_args(argv)
    dtypes = {"f16": np.float16, "f32": np.float32}
    ng = NervanaGPU(stochastic_round=False, bench=False)
    results = []
    for name in args.nets.split(","):
        for d in args.dtypes.split(","):
            title = "%s (dtype=%s, N=%d)" % (name, np.dtype(dtypes[d]).name, _NETS[name]["N"])
            print("------------------------------------------------")
            print("Benchmarking: " + title)
            print("------------------------------------------------")
            r = run_network(ng, name, dtypes[d], loops=args.loops, zeros=args.zeros, verbose=not args.quiet, warmup=args.warmup,
                            fold_relu=args.fold_relu)
            results.append(r)
            print("---------------------------------------------")
            print(title + " Results:")
            print("---------------------------------------------")
            print("Avg(%d) fprop: %8.3f msecs %.3f gflops" % (args.loops, r["fprop_ms"], r["fprop_gflops"]))
            print("Avg(%d) bprop: %8.3f msecs %.3f gflops" % (args.loops, r["bprop_ms"], r["bprop_gflops"]))
            print("Avg(%d) total: %8.3f msecs %.3f gflops" % (args.loops, r["total_ms"], r["total_gflops"]))
            if "published_titan_x_ms" in r:
                p = r["published_titan_x_ms"]
                print("reference on GTX Titan X: fprop %.3f bprop %.3f total %.3f msecs  (x%.1f)\n"
                      % (p["fprop"], p["bprop"], p["total"], r["speedup_vs_published_total"]))
            sys.stdout.flush()
    if args.json:
        with open(args.json, "w") as f:
            json.dump(results, f, indent=1)
    return results


if __name__ == "__main__":
    main()
