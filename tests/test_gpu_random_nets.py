"""Randomly composed layer graphs (chains with residual and concatenation edges) against the CPU oracle, through the C ABI: shapes, strides, paddings, activations
and layer types are drawn from a seeded generator, so that halo handling, tile selection at odd sizes, buffer reuse
between unrelated layers and the hand-over of activations are exercised in combinations no hand-written case lists.
Every layer is compared on identical inputs (fp16 storage) or along the free-running chain (fp32 storage)."""
import numpy as np
import pytest

import fyusenet_amd as fa
from fyusenet_amd import prng
from oracle import oracle as O
from util import conv_block, rel_l2

pytestmark = pytest.mark.gpu
TOL = {fa.STORAGE_F32: 1e-4, fa.STORAGE_F16: 2e-3}
A, T = fa.ActType, fa.LayerType


def _random_chain(seed):
    """Returns (input shape, [spec]) where spec = dict(kind, params...), output shape tracked along the chain."""
    rng = np.random.RandomState(seed)
    c, h, w = int(rng.choice([3, 4, 8, 16, 24])), int(rng.randint(6, 30)), int(rng.randint(6, 30))
    shape0 = (c, h, w)
    specs = []
    for _ in range(int(rng.randint(4, 9))):
        kinds = ["conv", "conv", "conv", "pool", "bn", "func", "scale"]
        if c >= 2:
            kinds.append("dw")
        if h <= 16 and w <= 16:
            kinds.append("tconv")
        if c <= 64:
            kinds.append("transpose")
        if specs:
            kinds += ["resconv", "resconv"]
            if len(specs) >= 2 and specs[-2]["out"][1:] == (h, w) and c + specs[-2]["out"][0] <= 128:
                kinds += ["cat", "cat"]
        kind = str(rng.choice(kinds))
        act = [A.NONE, A.RELU, A.CLIP, A.LEAKY_RELU][int(rng.randint(0, 4))]
        s = {"kind": kind, "act": act, "cin": c, "h": h, "w": w}
        if kind == "conv":
            s["k"] = int(rng.choice([1, 3, 3, 5]))
            s["dil"] = int(rng.choice([1, 2])) if s["k"] == 3 else 1
            s["stride"] = int(rng.choice([1, 2])) if min(h, w) >= 4 else 1
            s["cout"] = int(rng.choice([3, 8, 16, 33, 64]))
            s["bn"] = bool(rng.randint(0, 2))
            s["pad_in"] = (s["k"] - 1) // 2 * s["dil"]
            c, h, w = s["cout"], h // s["stride"], w // s["stride"]
        elif kind == "resconv":       # y = conv3x3(x) (+BN) + [ReLU](x): both ports read the previous layer
            s["bn"] = bool(rng.randint(0, 2))
            s["res_relu"] = bool(rng.randint(0, 2))
            s["pad_in"] = 1
        elif kind == "cat":           # concat(previous layer, the layer before it)
            s["other"] = len(specs) - 2
            s["pad_in"] = int(rng.randint(0, 2))
            c = c + specs[-2]["out"][0]
        elif kind == "dw":
            s["stride"] = int(rng.choice([1, 2])) if min(h, w) >= 4 else 1
            s["bn"] = bool(rng.randint(0, 2))
            s["pad_in"] = 1
            h, w = h // s["stride"], w // s["stride"]
        elif kind == "tconv":
            s["k"] = int(rng.choice([2, 3]))
            s["crop"] = int(rng.randint(0, 2)) if s["k"] == 3 else 0
            s["cout"] = int(rng.choice([4, 8, 24]))
            s["pad_in"] = 1
            c, h, w = s["cout"], 2 * h + s["k"] - 2 - s["crop"], 2 * w + s["k"] - 2 - s["crop"]
        elif kind == "pool":
            s["op"] = str(rng.choice(["max", "avg"]))
            s["pool"] = int(rng.choice([2, 3])) if min(h, w) >= 4 else 2
            if min(h, w) < 2:
                s["kind"] = kind = "bn"
                s["pad_in"] = int(rng.randint(0, 2))
            else:
                s["stride"] = 2 if s["pool"] == 2 else int(rng.choice([1, 2]))
                s["pad_in"] = 1 if s["pool"] == 3 else 0
                h, w = h // s["stride"], w // s["stride"]
        elif kind == "scale":
            s["pad_in"] = int(rng.randint(0, 2))
            s["linear"] = bool(rng.randint(0, 2))
            if max(h, w) <= 20 and rng.randint(0, 2):
                s["up"], s["down"] = 2, 1
                h, w = 2 * h, 2 * w
            elif min(h, w) >= 4:
                s["up"], s["down"] = 1, 2
                h, w = h // 2, w // 2
            else:
                s["up"], s["down"] = 1, 1
        elif kind == "func":
            s["fn"] = str(rng.choice(["sigmoid", "tanh", "arith", "relu"]))
            s["pad_in"] = int(rng.randint(0, 2))
        elif kind == "transpose":
            s["pad_in"] = 0
            h, w = w, h
        if kind == "bn":
            s.setdefault("pad_in", int(rng.randint(0, 2)))
        if h < 1 or w < 1:
            break
        s["out"] = (c, h, w)
        specs.append(s)
    return shape0, specs, int(rng.randint(0, 2))


def _builder(i, s, pad_out, specs=None, pads=None):
    no, name = i + 1, "%s%d" % (s["kind"], i + 1)
    cin, h, w = s["cin"], s["h"], s["w"]
    k = s["kind"]
    if k == "resconv":
        b = fa.ConvLayerBuilder(3, name).type(T.CONVOLUTION2D).shape(cin, h, w, cin)
        if s["bn"]:
            b.postfixNorm(fa.NormType.BATCHNORM)
        b.residual(A.RELU if s["res_relu"] else A.NONE, s["bn"]).residualPadding(s["pad_in"])
        weights = conv_block(1000 + 17 * no, cin, 3, cin, bn=s["bn"])
    elif k == "cat":
        o = s["other"]
        b = fa.ConcatLayerBuilder(name).input(cin, s["pad_in"]).input(specs[o]["out"][0], pads[o])
        b.size(w, h)
        b.outputChannels_ = s["out"][0]
        weights = None
    elif k in ("conv", "dw", "tconv"):
        kk = 3 if k == "dw" else s["k"]
        cout = cin if k == "dw" else s["cout"]
        b = fa.ConvLayerBuilder(kk, name).type(T.TRANSCONVOLUTION2D if k == "tconv" else T.CONVOLUTION2D).shape(cout, h, w, cin)
        if k == "dw":
            b.groupSize(cin)
        if k == "tconv":
            b.upsample(2).crop(s["crop"])
        else:
            b.downsample(s["stride"]).dilation(s.get("dil", 1))
            if s["bn"]:
                b.postfixNorm(fa.NormType.BATCHNORM)
        weights = conv_block(1000 + 17 * no, cout, kk, cin, bn=s.get("bn", False), depthwise=(k == "dw"))
    elif k == "pool":
        b = fa.PoolLayerBuilder(fa.PoolLayerBuilder.POOL_MAX if s["op"] == "max" else fa.PoolLayerBuilder.POOL_AVG, name)
        b.shape(cin, h, w, cin).poolSize(s["pool"]).downsample(s["stride"])
        weights = None
    elif k == "bn":
        b = fa.GPULayerBuilder(name).type(T.BATCHNORM).shape(cin, h, w, cin)
        weights = np.concatenate([prng.uniform(2000 + no, (cin,), 0.5, 1.5), prng.normal(3000 + no, (cin,), 0, 0.2)]).astype(np.float32)
    elif k == "scale":
        b = fa.ScaleLayerBuilder(name).shape(cin, h, w, cin).upsample(s["up"]).downsample(s["down"])
        b.scaleType(fa.ScalingType.LINEAR if s["linear"] else fa.ScalingType.NEAREST)
        weights = None
    elif k == "func":
        if s["fn"] == "arith":
            b = fa.SingletonArithLayerBuilder(name, fa.ArithType.MUL).operand(0.75).shape(cin, h, w, cin)
        else:
            b = fa.GPULayerBuilder(name).type({"sigmoid": T.SIGMOID, "tanh": T.TANH, "relu": T.RELU}[s["fn"]]).shape(cin, h, w, cin)
        weights = None
    else:
        b = fa.TransposeLayerBuilder(name).shape(cin, h, w, cin)
        weights = None
    b.number(no).inputPadding(s["pad_in"]).outputPadding(pad_out).deep()
    act = s["act"]
    if k == "cat" and act == A.LEAKY_RELU:
        act = A.RELU
    if k in ("pool",) and s["op"] == "max" and act in (A.CLIP, A.LEAKY_RELU):
        act = A.RELU      # the zero halo of a max-pool only equals -inf padding under a non-negative activation
    b.prefixAct(act)
    if act == A.CLIP:
        b.clip(-0.5, 1.5)
    if act == A.LEAKY_RELU:
        b.leakyReLU(0.2)
    return b, weights


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("seed", [sd for sd in range(40) if _random_chain(sd)[1]])   # (seeds whose chain has a layer)
def test_random_chain(seed, storage):
    shape0, specs, last_pad = _random_chain(seed)
    built = []
    pads = [specs[i + 1]["pad_in"] if i + 1 < len(specs) else last_pad for i in range(len(specs))]   # output padding per layer
    for i, s in enumerate(specs):
        built.append(_builder(i, s, pads[i], specs, pads))
    print("seed", seed, "input", shape0, [(s["kind"], s["out"]) for s in specs], flush=True)

    class Net(fa.NeuralNetwork):
        def buildLayers(self, f):
            for b, _ in built:
                b.push(f)

        def connectLayers(self, layers, bm):
            for i in range(1, len(built)):
                bm.connectLayers(layers[i], layers[i + 1], 0)
                if specs[i]["kind"] == "resconv":
                    bm.connectLayers(layers[i], layers[i + 1], 1)
                if specs[i]["kind"] == "cat":
                    bm.connectLayers(layers[specs[i]["other"] + 1], layers[i + 1], 1)

        def initializeWeights(self, layers):
            for b, w in built:
                if w is None:
                    continue
                if int(b.type_) == int(T.BATCHNORM):
                    layers[b.number_].loadScaleAndBias(w, 0)
                else:
                    layers[b.number_].loadWeightsAndBiases(w, 0)

    x = prng.uniform(5000 + seed, shape0, -1.5, 1.5)
    outs = {}
    for reuse in (True, False):
        net = Net(storage)
        net.setup(reuseBuffers=reuse)
        net.layers[1].setInput(x, 0)
        net.forward()
        net.finish()
        got = {lyr.number: lyr.copyResult() for lyr in net.layers}
        if reuse:
            # with buffer sharing only the last tensor is guaranteed to survive the pass
            outs["reuse"] = got[len(built)]
            net.cleanup()
            continue
        desc = net.describe()
        ref = O.run_network(desc, {(1, 0): x})
        forced = O.run_network(desc, {(1, 0): x}, forced=got) if storage == fa.STORAGE_F16 else ref
        for lyr in net.layers:
            e = rel_l2(got[lyr.number], forced[lyr.number])
            print("   %2d %-12s %-70s %.2e" % (lyr.number, lyr.name, lyr.kernelInfo()[:70], e), flush=True)
            assert got[lyr.number].shape == tuple(specs[lyr.number - 1]["out"])
            assert e <= TOL[storage], (seed, lyr.name, e)
        assert np.array_equal(outs["reuse"], got[len(built)])       # buffer sharing does not change a bit
        net.cleanup()


def _random_shallow_chain(seed):
    """Shallow layers only: convolutions whose halo may be narrower than the kernel reaches (edge repeat or zero halo),
    residual convolutions, fractional-step convolutions, batch norm and function layers."""
    rng = np.random.RandomState(10_000 + seed)
    c, h, w = int(rng.choice([3, 4, 12, 20])), int(rng.randint(4, 20)), int(rng.randint(4, 20))
    shape0, specs = (c, h, w), []
    for _ in range(int(rng.randint(3, 7))):
        kinds = ["conv", "conv", "frac", "bn", "func"] + (["resconv"] if specs else [])
        if h * w > 1600:
            kinds = [k for k in kinds if k != "frac"] or ["conv"]
        kind = str(rng.choice(kinds))
        act = [A.NONE, A.RELU, A.CLIP, A.LEAKY_RELU][int(rng.randint(0, 4))]
        s = {"kind": kind, "act": act, "cin": c, "h": h, "w": w}
        if kind == "conv":
            s["k"] = int(rng.choice([1, 3, 3, 5, 9]))
            s["stride"] = 2 if (min(h, w) >= 4 and h % 2 == 0 and w % 2 == 0 and rng.randint(0, 3) == 0) else 1
            s["cout"] = int(rng.choice([3, 12, 20, 40]))
            s["bn"] = bool(rng.randint(0, 2))
            s["pad_in"] = int(rng.randint(0, (s["k"] - 1) // 2 + 1))     # 0 .. r: anything short of r repeats or pads
            c, h, w = s["cout"], h // s["stride"], w // s["stride"]
        elif kind == "resconv":
            s["bn"] = bool(rng.randint(0, 2))
            s["res_relu"] = bool(rng.randint(0, 2))
            s["pad_in"] = int(rng.randint(0, 2))
        elif kind == "frac":
            s["k"] = int(rng.choice([3, 3, 5, 7, 9]))
            s["inv"] = int(rng.choice([2, 2, 4]))
            s["stride"] = int(rng.choice([1, 2]))
            s["cout"] = int(rng.choice([3, 12, 20]))
            s["bn"] = bool(rng.randint(0, 2))
            s["pad_in"] = int(rng.randint(0, 3))
            c, h, w = s["cout"], h * s["inv"] // s["stride"], w * s["inv"] // s["stride"]
        elif kind == "func":
            s["fn"] = str(rng.choice(["sigmoid", "tanh", "arith", "relu"]))
            s["pad_in"] = int(rng.randint(0, 2))
        else:
            s["pad_in"] = int(rng.randint(0, 2))
        s["out"] = (c, h, w)
        specs.append(s)
    return shape0, specs, int(rng.randint(0, 2))


def _shallow_builder(i, s, pad_out):
    no, name = i + 1, "%s%d" % (s["kind"], i + 1)
    cin, h, w, k = s["cin"], s["h"], s["w"], s["kind"]
    weights = None
    if k == "resconv":
        b = fa.ConvLayerBuilder(3, name).type(T.CONVOLUTION2D).shape(cin, h, w, cin)
        if s["bn"]:
            b.postfixNorm(fa.NormType.BATCHNORM)
        b.residual(A.RELU if s["res_relu"] else A.NONE, s["bn"]).residualPadding(s["pad_in"])
        weights = conv_block(4000 + 17 * no, cin, 3, cin, bn=s["bn"])
    elif k in ("conv", "frac"):
        b = fa.ConvLayerBuilder(s["k"], name).type(T.CONVOLUTION2D if k == "conv" else T.FRACCONVOLUTION2D).shape(s["cout"], h, w, cin)
        b.downsample(s["stride"])
        if k == "frac":
            b.sourceStep(1.0 / s["inv"])
        if s["bn"]:
            b.postfixNorm(fa.NormType.BATCHNORM)
        weights = conv_block(4000 + 17 * no, s["cout"], s["k"], cin, bn=s["bn"])
    elif k == "bn":
        b = fa.GPULayerBuilder(name).type(T.BATCHNORM).shape(cin, h, w, cin)
        weights = np.concatenate([prng.uniform(6000 + no, (cin,), 0.5, 1.5), prng.normal(7000 + no, (cin,), 0, 0.2)]).astype(np.float32)
    elif s["fn"] == "arith":
        b = fa.SingletonArithLayerBuilder(name, fa.ArithType.MUL).operand(0.75).shape(cin, h, w, cin)
    else:
        b = fa.GPULayerBuilder(name).type({"sigmoid": T.SIGMOID, "tanh": T.TANH, "relu": T.RELU}[s["fn"]]).shape(cin, h, w, cin)
    b.number(no).inputPadding(s["pad_in"]).outputPadding(pad_out).prefixAct(s["act"])
    if s["act"] == A.CLIP:
        b.clip(-0.5, 1.5)
    if s["act"] == A.LEAKY_RELU:
        b.leakyReLU(0.2)
    return b, weights


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("seed", range(24))
def test_random_shallow_chain(seed, storage):
    shape0, specs, last_pad = _random_shallow_chain(seed)
    pads = [specs[i + 1]["pad_in"] if i + 1 < len(specs) else last_pad for i in range(len(specs))]
    built = [_shallow_builder(i, s, pads[i]) for i, s in enumerate(specs)]
    print("seed", seed, "input", shape0, [(s["kind"], s.get("k"), s["pad_in"], s["out"]) for s in specs], flush=True)

    class Net(fa.NeuralNetwork):
        def buildLayers(self, f):
            for b, _ in built:
                b.push(f)

        def connectLayers(self, layers, bm):
            for i in range(1, len(built)):
                bm.connectLayers(layers[i], layers[i + 1], 0)
                if specs[i]["kind"] == "resconv":
                    bm.connectLayers(layers[i], layers[i + 1], 1)

        def initializeWeights(self, layers):
            for b, w in built:
                if w is None:
                    continue
                if int(b.type_) == int(T.BATCHNORM):
                    layers[b.number_].loadScaleAndBias(w, 0)
                else:
                    layers[b.number_].loadWeightsAndBiases(w, 0)

    x = prng.uniform(8000 + seed, shape0, -1.5, 1.5)
    net = Net(storage)
    net.setup(reuseBuffers=False)
    net.layers[1].setInput(x, 0)
    net.forward()
    net.finish()
    got = {lyr.number: lyr.copyResult() for lyr in net.layers}
    desc = net.describe()
    ref = O.run_network(desc, {(1, 0): x})
    forced = O.run_network(desc, {(1, 0): x}, forced=got) if storage == fa.STORAGE_F16 else ref
    for lyr in net.layers:
        e = rel_l2(got[lyr.number], forced[lyr.number])
        print("   %2d %-12s %-70s %.2e" % (lyr.number, lyr.name, lyr.kernelInfo()[:70], e), flush=True)
        assert got[lyr.number].shape == tuple(specs[lyr.number - 1]["out"])
        assert e <= TOL[storage], (seed, lyr.name, e)
    net.cleanup()
