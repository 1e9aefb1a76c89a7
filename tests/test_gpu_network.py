"""Whole-network driver (Layer.create, shared delta / update buffers, fprop and
bprop loops of benchmarks/convnet-benchmarks.py:250-403 of the reference):
every layer's forward output, data gradient and weight gradient is checked
against the numpy oracle fed with the tensors the GPU layer actually received."""
import numpy as np
import pytest

import oracle as orc
from util import assert_fp16_within_ulp, assert_fp32_close, acc_atol

pytestmark = pytest.mark.gpu


def _small_net():
    from nervanagpu_amd.layers import DataLayer, ConvLayer, PoolLayer, FullLayer
    return [
        {"layer": DataLayer, "N": 16, "C": 3, "H": 20, "W": 20},
        {"layer": ConvLayer, "K": 16, "R": 3, "S": 3, "pad_h": 1, "pad_w": 1},
        {"layer": PoolLayer, "op": "max", "R": 2, "S": 2},
        {"layer": ConvLayer, "K": 32, "R": 3, "S": 3, "pad_h": 1, "pad_w": 1, "str_h": 2, "str_w": 2},
        {"layer": PoolLayer, "op": "max", "R": 3, "S": 3, "str_h": 2, "str_w": 2},
        {"layer": FullLayer, "nOut": 64},
        {"layer": FullLayer, "nOut": 16},
    ]


def _check(out, ref, dtype, what, absacc):
    if np.dtype(dtype) == np.float16:
        assert_fp16_within_ulp(out, ref, 1.0, what, acc_atol(absacc))
    else:
        assert_fp32_close(out, ref, 1e-5, what)


def _conv_args(layer):
    return dict(padding=layer.padding, strides=layer.strides)


def _check_fprop(layer, x, got, dtype, what):
    """one layer's forward output against the oracle on the input x it received"""
    from nervanagpu_amd.layers import ConvLayer, PoolLayer, FullLayer
    if type(layer) is ConvLayer:
        F = layer.weights.get().astype(np.float32)
        x = x.reshape(layer.dimI)
        ref = orc.ref_conv_fprop(x, F, relu=True, **_conv_args(layer))
        absdot = orc.ref_conv_fprop(np.abs(x), np.abs(F), **_conv_args(layer))
        _check(got, ref, dtype, what, absdot)
    elif type(layer) is PoolLayer:
        ref = orc.ref_pool_fprop(x.reshape(layer.dimI), layer.op, layer.JTRS, layer.padding, layer.strides)
        if layer.op == "max":
            assert np.array_equal(got.astype(np.float32), ref.astype(dtype).astype(np.float32)), what
        else:
            _check(got, ref, dtype, what, 0.0)
    elif type(layer) is FullLayer:
        W = layer.weights.get().astype(np.float32)
        x2 = x.reshape(layer.dimI)
        _check(got, orc.ref_dot(W, x2, relu=True), dtype, what, np.abs(W) @ np.abs(x2))


def _bprop_checked(layer, err, dtype, what):
    """run layer.bprop(err) and check its data and weight gradients against the
    oracle fed with the error, activations and inputs the layer held"""
    from nervanagpu_amd.layers import ConvLayer, PoolLayer
    e_in = err.get().astype(np.float32)
    act = layer.fprop_out.get().astype(np.float32)
    x = layer.fprop_in.get().astype(np.float32)
    out = layer.bprop(err)
    if type(layer) is PoolLayer:
        ref = orc.ref_pool_bprop(x, e_in.reshape(layer.dimO), layer.op, layer.JTRS, layer.padding, layer.strides)
        _check(out.get(), ref, dtype, what, 0.0)
        return out
    # relu derivative applied in place by the layer, then rounded to the layer dtype
    em = (e_in.reshape(act.shape) * (act > 0)).astype(dtype).astype(np.float32)
    if type(layer) is ConvLayer:
        F = layer.weights.get().astype(np.float32)
        if layer.bprop_out is not None:
            ref = orc.ref_conv_bprop(F, em, layer.dimI, **_conv_args(layer))
            absdot = orc.ref_conv_bprop(np.abs(F), np.abs(em), layer.dimI, **_conv_args(layer))
            _check(out.get(), ref, dtype, what + " dI", absdot)
        refu = orc.ref_conv_update(x, em, layer.dimF, **_conv_args(layer))
        absu = orc.ref_conv_update(np.abs(x), np.abs(em), layer.dimF, **_conv_args(layer))
        _check(layer.updat_out.get(), refu, layer.updat_out.dtype, what + " dF", absu)
    else:
        W = layer.weights.get().astype(np.float32)
        em2 = em.reshape(layer.dimO)
        _check(out.get(), orc.ref_dot(W.T, em2), dtype, what + " dI", np.abs(W.T) @ np.abs(em2))
        x2 = x.reshape(layer.dimI)
        _check(layer.updat_out.get(), orc.ref_dot(em2, x2.T), layer.updat_out.dtype, what + " dW",
               np.abs(em2) @ np.abs(x2.T))
    return out


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_network_fprop_bprop_layerwise(ng, dtype):
    from nervanagpu_amd import convnet_benchmarks as cb
    layers = cb.build_network(ng, _small_net(), dtype, seed=5)

    # ---- forward: each layer against the oracle on the input it received
    propagation = None
    for li, layer in enumerate(layers):
        x = None if propagation is None else propagation.get().astype(np.float32)
        propagation = layer.fprop(propagation)
        if li:
            _check_fprop(layer, x, propagation.get(), dtype, "fprop layer %d %s" % (li, layer))

    # ---- backward: the final activations serve as the error, as in the reference loop
    for li in range(len(layers) - 1, 0, -1):
        propagation = _bprop_checked(layers[li], propagation, dtype, "bprop layer %d %s" % (li, layers[li]))


def _inception_net():
    from nervanagpu_amd.layers import DataLayer, FullLayer
    from nervanagpu_amd import convnet_benchmarks as cb
    return [
        {"layer": DataLayer, "N": 16, "C": 8, "H": 12, "W": 12},
        cb._conv(16, 3, 1),
        cb._inception("incep1", ((16,), (8, 16), (8, 8), (8,))),
        cb._inception("incep2", ((0,), (8, 16), (8, 16), ("max", 0))),
        cb._conv(32, 2, 0, 2),
        cb._inception("incep2", ((8,), (8, 16), (8, 8), ("avg", 16))),
        cb._pool(6, 1, 0, "avg"),
        {"layer": FullLayer, "nOut": 16},
    ]


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_inception_network_layerwise(ng, dtype):
    """Inception layers (nervanagpu/layers.py:520-640 of the reference): branches
    read the module's input, their last layers write channel slices of the
    module's output; on the way back each branch takes its slice of the error
    and inner layers alternate between two more shared delta buffers."""
    from nervanagpu_amd import convnet_benchmarks as cb
    from nervanagpu_amd.layers import Inception
    layers = cb.build_network(ng, _inception_net(), dtype, seed=11)
    assert [type(l) is Inception for l in layers] == [False, False, True, True, False, True, False, False]
    assert [l.K for l in layers[2:6]] == [48, 16 + 16 + 48, 32, 48]

    propagation = None
    for li, layer in enumerate(layers):
        x = None if propagation is None else propagation.get().astype(np.float32)
        propagation = layer.fprop(propagation)
        if type(layer) is not Inception:
            if li:
                _check_fprop(layer, x, propagation.get(), dtype, "fprop layer %d %s" % (li, layer))
            continue
        k0, whole = 0, propagation.get()
        assert whole.shape == layer.dimO
        for pi, part in enumerate(layer.partitions):
            px = x
            for layer2 in part:
                got = layer2.fprop_out.get()
                _check_fprop(layer2, px, got, dtype, "fprop layer %d part %d %s" % (li, pi, layer2))
                px = got.astype(np.float32)
            # the branch tail is a channel slice of the module's output
            assert np.array_equal(whole[k0:k0 + part[-1].K].view(np.uint8), got.view(np.uint8))
            k0 += part[-1].K
        assert k0 == layer.K

    for li in range(len(layers) - 1, 0, -1):
        layer = layers[li]
        what = "bprop layer %d" % li
        if type(layer) is not Inception:
            propagation = _bprop_checked(layer, propagation, dtype, what + " %s" % layer)
            continue
        # the module's own loop, one checked layer at a time
        K = layer.K
        first = {}
        for pi in range(len(layer.partitions) - 1, -1, -1):
            part = layer.partitions[pi]
            err = propagation[K - part[-1].K:K, ...]
            K -= part[-1].K
            for layer2 in part[::-1]:
                err = _bprop_checked(layer2, err, dtype, what + " part %d %s" % (pi, layer2))
            assert err is layer.bprop_out
            first[pi] = err.get()
        # every branch writes the module's delta buffer; as in the reference the
        # last one run (the first branch) is what the layer below receives
        again = layer.bprop(propagation)
        assert again is layer.bprop_out
        assert np.array_equal(again.get().view(np.uint8), first[0].view(np.uint8))
        propagation = again


def _conv_pairs_net():
    from nervanagpu_amd.layers import DataLayer, ConvLayer, PoolLayer, FullLayer
    return [
        {"layer": DataLayer, "N": 16, "C": 3, "H": 16, "W": 16},
        {"layer": ConvLayer, "K": 16, "R": 3, "S": 3, "pad_h": 1, "pad_w": 1},
        {"layer": ConvLayer, "K": 24, "R": 3, "S": 3, "pad_h": 1, "pad_w": 1},
        {"layer": PoolLayer, "op": "max", "R": 2, "S": 2},
        {"layer": ConvLayer, "K": 32, "R": 3, "S": 3, "pad_h": 1, "pad_w": 1},
        {"layer": ConvLayer, "K": 32, "R": 1, "S": 1},
        {"layer": ConvLayer, "K": 16, "R": 3, "S": 3, "str_h": 2, "str_w": 2},   # strided: not folded
        {"layer": PoolLayer, "op": "avg", "R": 3, "S": 3},                       # average: not folded
        {"layer": FullLayer, "nOut": 16},
    ]


@pytest.mark.parametrize("net,pairs", [(_small_net, 2), (_conv_pairs_net, 3)])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_folded_rectifier_derivatives_give_the_same_network(ng, dtype, net, pairs):
    """fold_relu_derivatives: max pooling and unit-stride convolution layers above
    rectified layers apply the rectifier derivative themselves; every gradient the
    rectified layers compute must equal the reference flow's (separate
    elementwise pass)."""
    from nervanagpu_amd import convnet_benchmarks as cb
    from nervanagpu_amd.layers import PoolLayer

    def run(fold):
        layers = cb.build_network(ng, net(), dtype, seed=5, fold_relu=fold)
        propagation = None
        for layer in layers:
            propagation = layer.fprop(propagation)
        grads = []
        for layer in layers[:0:-1]:
            propagation = layer.bprop(propagation)
            # what a layer hands down differs by design (masked now, or by the
            # layer below later, in place); what the layer below computes from
            # it must not: weight gradients, and data gradients after masking
            if layer.weights is not None:
                grads.append(layer.updat_out.get().copy())
        grads.append(None if propagation is None else propagation.get().copy())
        return layers, grads

    plain_layers, plain = run(False)
    folded_layers, folded = run(True)
    assert sum(l.relu_done_above for l in folded_layers) == pairs and not any(l.relu_done_above for l in plain_layers)
    assert len(plain) == len(folded)
    for a, b in zip(plain, folded):
        assert (a is None) == (b is None)
        if a is not None:
            assert np.array_equal(a, b)
