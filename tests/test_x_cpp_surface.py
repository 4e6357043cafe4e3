"""The C++ description surface (include/fynhip.hpp: builders, LayerFactory, CompiledLayers, BufferManager,
NeuralNetwork under the reference's names) through a program compiled with the host compiler only
(tests/cpp/surface_example.cpp)."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "cpp", "surface_example.cpp")
EXE = os.path.join(ROOT, "tests", "cpp", "_build", "surface_example")

# The hourglass of surface_example.cpp, row for row:
# (number, name, kind, kernel, cin, cout, shrink, stride, act, bn, pad_out, from, residual_from)
TABLE = [
    (0, "in", "up", 0, 3, 3, 1, 1, "none", False, 2, -1, -1),
    (1, "wide", "conv", 5, 3, 16, 1, 1, "none", True, 1, 0, -1),
    (2, "down", "conv", 3, 16, 32, 1, 2, "relu", True, 1, 1, -1),
    (3, "pair_a", "conv", 3, 32, 32, 2, 1, "relu", True, 1, 2, -1),
    (4, "pair_b", "conv", 3, 32, 32, 2, 1, "relu", True, 1, 3, 2),
    (5, "up", "tconv", 3, 32, 16, 2, 2, "relu", True, 0, 4, -1),
    (6, "mix", "conv", 1, 16, 8, 1, 1, "leaky", False, 0, 5, -1),
    (7, "out", "down", 0, 8, 8, 1, 1, "none", False, 0, 6, -1),
]
LEAK = 0.125


def test_cpp_surface_compiles_with_the_host_compiler(tmp_path):
    """Header and program compile as plain C++17 without warnings (no HIP, no torch in the interface)."""
    obj = tmp_path / "surface_example.o"
    r = subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", SRC, "-o", str(obj)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert obj.stat().st_size > 0


def _python_twin(width, height, stream):
    import fyusenet_amd as fa
    from fyusenet_amd.builders import ActType, ConvLayerBuilder, LayerType, NormType, UpDownLayerBuilder
    from fyusenet_amd.network import NeuralNetwork
    acts = {"none": ActType.NONE, "relu": ActType.RELU, "leaky": ActType.LEAKY_RELU}

    class Hourglass(NeuralNetwork):
        def buildLayers(self, factory):
            for (no, name, kind, k, cin, cout, shrink, stride, act, bn, pad_out, _src, res) in TABLE:
                h, w = height // shrink, width // shrink
                if kind in ("up", "down"):
                    b = UpDownLayerBuilder(UpDownLayerBuilder.UPLOAD if kind == "up" else UpDownLayerBuilder.DOWNLOAD, name)
                    b.shape(cout, h, w, cin).outputPadding(pad_out).number(no)
                    if kind == "down":
                        b.deep()
                else:
                    b = ConvLayerBuilder(k, name).shape(cout, h, w, cin).deep().inputPadding((k - 1) // 2).outputPadding(pad_out)
                    b.prefixAct(acts[act]).number(no)
                    if act == "leaky":
                        b.leakyReLU(LEAK)
                    if bn:
                        b.postfixNorm(NormType.BATCHNORM)
                    if kind == "tconv":
                        b.type(LayerType.TRANSCONVOLUTION2D).upsample(stride).crop(1)
                    else:
                        b.type(LayerType.CONVOLUTION2D).downsample(stride)
                    if res >= 0:
                        b.residual(ActType.RELU).residualPadding(pad_out)
                b.push(factory)

        def connectLayers(self, layers, bm):
            for row in TABLE:
                if row[11] >= 0:
                    bm.connectLayers(layers[row[11]], layers[row[0]], 0)
                if row[12] >= 0:
                    bm.connectLayers(layers[row[12]], layers[row[0]], 1)

        def initializeWeights(self, layers):
            at = 0
            for row in TABLE:
                n = _block_floats(row)
                if n:
                    layers[row[0]].loadWeightsAndBiases(stream, at)
                    at += n

    return Hourglass(fa.STORAGE_F32)


def _block_floats(row):
    (_no, _name, kind, k, cin, cout, *_rest) = row
    bn = row[9]
    return cout + cout * k * k * cin + (2 * cout if bn else 0) if kind in ("conv", "tconv") else 0


@pytest.mark.gpu
def test_cpp_program_matches_the_python_surface(tmp_path):
    """The program's own checks (known answers on constant images, the factory's error messages, ascending layer order,
    the frame pipeline, reloading weights, a pool of instances) and its network output, which must equal, bit for bit,
    what the same table gives through the Python surface with the same weight stream and input."""
    from fyusenet_amd import prng
    from util import conv_block
    assert os.path.exists(EXE), "tests/cpp/_build/surface_example is not built (run __graft_entry__.build())"
    width, height = 64, 48
    stream = np.concatenate([conv_block(900 + 4 * row[0], row[5], row[3], row[4], bn=row[9]) for row in TABLE if _block_floats(row)]).astype(np.float32)
    assert stream.size == sum(_block_floats(r) for r in TABLE)
    frame = prng.uniform(4242, (3, height, width), 0.0, 1.0)
    net = _python_twin(width, height, stream)
    net.setup()
    net.layers[0].setInput(frame, 0)
    net.forward()
    net.finish()
    want = net.getOutput(7)
    from oracle import oracle as O
    from util import rel_l2
    ref = O.run_network(net.describe(), {(0, 0): frame})[7]
    net.cleanup()
    assert rel_l2(want, ref) <= 1e-4   # fp32 storage
    assert want.shape == (8, height, width)
    stream.astype("<f4").tofile(tmp_path / "weights.bin")
    frame.astype("<f4").tofile(tmp_path / "input.bin")
    r = subprocess.run([EXE, str(tmp_path / "weights.bin"), str(tmp_path / "input.bin"), str(tmp_path / "output.bin"), str(width), str(height)],
                       capture_output=True, text=True, timeout=110)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stderr
    assert "0 check(s) failed" in r.stdout
    got = np.fromfile(tmp_path / "output.bin", dtype="<f4").reshape(8, height, width)
    assert np.array_equal(got, want)
    assert np.isfinite(got).all() and got.std() > 0
