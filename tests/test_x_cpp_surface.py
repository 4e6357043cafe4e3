"""The C++ description surface (include/fynhip.hpp: builders, LayerFactory, CompiledLayers, BufferManager,
NeuralNetwork with the reference's names) through a program written the way the reference's samples and unit tests are
written (tests/cpp/reference_style.cpp)."""
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "cpp", "reference_style.cpp")
EXE = os.path.join(ROOT, "tests", "cpp", "_build", "reference_style")


def test_cpp_surface_compiles_with_the_host_compiler(tmp_path):
    """Header and program compile as plain C++17 without warnings (no HIP, no torch in the interface)."""
    obj = tmp_path / "reference_style.o"
    r = subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", SRC, "-o", str(obj)],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert obj.stat().st_size > 0


@pytest.mark.gpu
def test_reference_style_cpp_program_matches_the_python_surface(tmp_path):
    """The program's own checks (the reference's known-answer patterns, the factory's error messages, the frame pipeline,
    reloading weights) and its style-net output, which must equal, bit for bit, what the same graph gives through the
    Python surface with the same weight stream and input."""
    import fyusenet_amd as fa
    from fyusenet_amd import prng, samples
    assert os.path.exists(EXE), "tests/cpp/_build/reference_style is not built (run __graft_entry__.build())"
    width, height = 64, 48
    net = samples.StyleNetSample(3, width, height, fa.STORAGE_F32)
    weights = net.synthetic_weights()
    rgb = prng.uniform(4242, (height, width, 3), 0.0, 1.0)
    net._weights = weights
    net.setup()
    net.layers[net.UPLOAD].setInput(rgb, 0, fa.capi.ORDER_GPU_SHALLOW)
    net.forward()
    net.finish()
    want = net.getOutput(net.DOWNLOAD, fa.capi.ORDER_GPU_SHALLOW)
    net.cleanup()
    assert want.shape == (height, width, 4)
    weights.astype("<f4").tofile(tmp_path / "weights.bin")
    rgb.astype("<f4").tofile(tmp_path / "input.bin")
    r = subprocess.run([EXE, str(tmp_path / "weights.bin"), str(tmp_path / "input.bin"), str(tmp_path / "output.bin"), str(width), str(height)],
                       capture_output=True, text=True, timeout=110)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, r.stderr
    assert "0 check(s) failed" in r.stdout and "fractional step 1/4" in r.stdout
    got = np.fromfile(tmp_path / "output.bin", dtype="<f4").reshape(height, width, 4)
    assert np.array_equal(got, want)
    assert np.all(got[..., :3] > 0) and np.all(got[..., :3] < 1) and not np.any(got[..., 3])
