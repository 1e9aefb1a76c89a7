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


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_network_fprop_bprop_layerwise(ng, dtype):
    from nervanagpu_amd import convnet_benchmarks as cb
    from nervanagpu_amd.layers import ConvLayer, PoolLayer, FullLayer
    layers = cb.build_network(ng, _small_net(), dtype, seed=5)

    # ---- forward: each layer against the oracle on the input it received
    propagation = None
    for li, layer in enumerate(layers):
        x = None if propagation is None else propagation.get().astype(np.float32)
        propagation = layer.fprop(propagation)
        got = propagation.get()
        what = "fprop layer %d %s" % (li, layer)
        if type(layer) is ConvLayer:
            F = layer.weights.get().astype(np.float32)
            ref = orc.ref_conv_fprop(x, F, relu=True, **_conv_args(layer))
            absdot = orc.ref_conv_fprop(np.abs(x), np.abs(F), **_conv_args(layer))
            _check(got, ref, dtype, what, absdot)
        elif type(layer) is PoolLayer:
            ref = orc.ref_pool_fprop(x.reshape(layer.dimI), layer.op, layer.JTRS, layer.padding, layer.strides)
            assert np.array_equal(got.astype(np.float32), ref.astype(dtype).astype(np.float32)), what
        elif type(layer) is FullLayer:
            W = layer.weights.get().astype(np.float32)
            x2 = x.reshape(layer.dimI)
            _check(got, orc.ref_dot(W, x2, relu=True), dtype, what, np.abs(W) @ np.abs(x2))

    # ---- backward: the final activations serve as the error, as in the reference loop
    for li in range(len(layers) - 1, 0, -1):
        layer = layers[li]
        e_in = propagation.get().astype(np.float32)
        act = layer.fprop_out.get().astype(np.float32)
        x = layer.fprop_in.get().astype(np.float32)
        propagation = layer.bprop(propagation)
        what = "bprop layer %d %s" % (li, layer)
        if type(layer) is PoolLayer:
            ref = orc.ref_pool_bprop(x, e_in.reshape(layer.dimO), layer.op, layer.JTRS, layer.padding, layer.strides)
            _check(propagation.get(), ref, dtype, what, 0.0)
            continue
        # relu derivative applied in place by the layer, then rounded to the layer dtype
        em = (e_in.reshape(act.shape) * (act > 0)).astype(dtype).astype(np.float32)
        if type(layer) is ConvLayer:
            F = layer.weights.get().astype(np.float32)
            if layer.bprop_out is not None:
                ref = orc.ref_conv_bprop(F, em, layer.dimI, **_conv_args(layer))
                absdot = orc.ref_conv_bprop(np.abs(F), np.abs(em), layer.dimI, **_conv_args(layer))
                _check(propagation.get(), ref, dtype, what + " dI", absdot)
            refu = orc.ref_conv_update(x, em, layer.dimF, **_conv_args(layer))
            absu = orc.ref_conv_update(np.abs(x), np.abs(em), layer.dimF, **_conv_args(layer))
            _check(layer.updat_out.get(), refu, layer.updat_out.dtype, what + " dF", absu)
        else:
            W = layer.weights.get().astype(np.float32)
            em2 = em.reshape(layer.dimO)
            _check(propagation.get(), orc.ref_dot(W.T, em2), dtype, what + " dI", np.abs(W.T) @ np.abs(em2))
            x2 = x.reshape(layer.dimI)
            _check(layer.updat_out.get(), orc.ref_dot(em2, x2.T), layer.updat_out.dtype, what + " dW",
                   np.abs(em2) @ np.abs(x2.T))
