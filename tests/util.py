"""Shared helpers of the test-suite."""
import itertools

import numpy as np
import pytest

from fyusenet_amd import prng


def combos(runs, **axes):
    """Arguments for pytest.mark.parametrize: the combinations of the named axes that runs(**combination) accepts, so
    that a test is generated only where it has something to run (instead of being generated and skipped).
    axes: name=(values, id function)."""
    names = list(axes)
    out = []
    for vals in itertools.product(*[axes[n][0] for n in names]):
        if runs(**dict(zip(names, vals))):
            out.append(pytest.param(*vals, id="-".join(axes[n][1](v) for n, v in zip(names, vals))))
    return ",".join(names), out


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    den = np.linalg.norm(b.ravel())
    if den == 0:
        return float(np.linalg.norm(a.ravel()))
    return float(np.linalg.norm((a - b).ravel()) / den)


def conv_block(seed, cout, k, cin, bn=False, depthwise=False):
    """Weight block in the reference's .dat order: [bias][W][bnScale][bnBias]; He-normal weights,
    bias ~ N(0, 0.01), BN scale ~ U(0.5, 1.5), BN bias ~ N(0, 0.1)."""
    if depthwise:
        w = prng.he_normal(seed, (cin * k * k,), k * k)
    else:
        w = prng.he_normal(seed, (cout * k * k * cin,), k * k * cin)
    parts = [prng.normal(seed + 1, (cout,), 0.0, 0.01), w]
    if bn:
        parts += [prng.uniform(seed + 2, (cout,), 0.5, 1.5), prng.normal(seed + 3, (cout,), 0.0, 0.1)]
    return np.concatenate(parts).astype(np.float32)


def make_single_layer_net(builder, storage, weights=None, scale_bias=None, reuse=True):
    """A network of one layer whose input ports are fed from the host, as the reference's layer unit
    tests do (unit_tests/layertestbase.cpp:208-417)."""
    import fyusenet_amd as fa

    class _Net(fa.NeuralNetwork):
        def buildLayers(self, factory):
            builder.push(factory)

        def connectLayers(self, layers, bm):
            pass

        def initializeWeights(self, layers):
            lyr = layers[builder.number_]
            if weights is not None:
                lyr.loadWeightsAndBiases(weights, 0)
            if scale_bias is not None:
                lyr.loadScaleAndBias(scale_bias, 0)

    net = _Net(storage)
    net.setup(reuseBuffers=reuse)
    return net


def run_single(builder, storage, inputs, weights=None, scale_bias=None):
    """inputs: list of CHW arrays per port. Returns the layer's CHW output."""
    net = make_single_layer_net(builder, storage, weights, scale_bias)
    lyr = net.layers[builder.number_]
    for port, x in enumerate(inputs):
        lyr.setInput(x, port)
    net.forward()
    net.finish()
    out = lyr.copyResult()
    info = lyr.kernelInfo()
    net.cleanup()
    return out, info


def oracle_single(builder, storage, inputs, weights=None):
    from oracle import oracle as O
    desc = {"layers": [{"builder": builder, "number": builder.number_, "weights": weights}], "connections": [], "storage": storage}
    feeds = {(builder.number_, p): x for p, x in enumerate(inputs)}
    return O.run_network(desc, feeds)[builder.number_]
