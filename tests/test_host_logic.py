"""CPU-only checks: the C-ABI library loads and exports every declared symbol, the ctypes struct
matches the header, builders compose flags like LayerBuilderTempl::getFlags, and the validation
errors of the reference's factory are raised without touching a GPU."""
import ctypes
import os
import re

import pytest

import fyusenet_amd as fa
from fyusenet_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "fynhip.h")).read()
    declared = set(re.findall(r"\b(fyn_[a-z_]+)\s*\(", header))
    assert declared == set(capi.SYMBOLS), declared ^ set(capi.SYMBOLS)
    lib = capi.lib()
    for name in declared:
        assert getattr(lib, name) is not None


def test_desc_struct_layout_matches_header():
    # 4-byte fields only, no padding: size must equal the sum of the members
    d = capi.LayerDesc()
    assert ctypes.sizeof(d) == 4 * 3 + 64 + 4 * (1 + 4 + 3 + 2 + 2 + 3 + 1 + 2 + 1 + 2 + 1 + 1) + 12 * 8 + 4 + 4 * 7
    # member names and order as the header declares them
    import re
    text = open(os.path.join(ROOT, "include", "fynhip.h")).read()
    body = text[text.index("typedef struct fyn_layer_desc {"):text.index("} fyn_layer_desc;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S).split("{", 1)[1]
    body = re.sub(r"struct\s*\{[^}]*\}", "struct_t", body)
    names = []
    for decl in body.split(";"):
        decl = decl.strip()
        if not decl:
            continue
        for part in decl.split(None, 1)[1].split(","):
            names.append(re.sub(r"\[.*", "", part).strip())
    assert names == [f[0] for f in capi.LayerDesc._fields_]


def test_flags_follow_getflags():
    b = fa.ConvLayerBuilder(3, "c").prefixAct(fa.ActType.RELU).postfixNorm(fa.NormType.BATCHNORM).deep().residual(fa.ActType.RELU, True)
    f = b.getFlags()
    assert f == (fa.LayerFlags.PRE_RELU | fa.LayerFlags.POST_BATCHNORM | fa.LayerFlags.DEEP | fa.LayerFlags.RESIDUAL_INPUT |
                 fa.LayerFlags.RELU_ON_RESIDUAL | fa.LayerFlags.BATCHNORM_ON_RESIDUAL)
    assert fa.ConvLayerBuilder(1, "c").prefixAct(fa.ActType.CLIP).getFlags() == fa.LayerFlags.PRE_CLIP
    assert fa.ConvLayerBuilder(1, "c").prefixAct(fa.ActType.LEAKY_RELU).getFlags() == fa.LayerFlags.PRE_RELU
    with pytest.raises(fa.FynException):
        fa.ConvLayerBuilder(1, "c").residual(fa.ActType.CLIP)
    with pytest.raises(fa.FynException):
        fa.ConvLayerBuilder(1, "c").prefixAct(fa.ActType.SIGMOID).getFlags()
    p = fa.PoolLayerBuilder(fa.PoolLayerBuilder.POOL_AVG, "p")
    with pytest.raises(fa.FynException):
        p.global_pool()  # size must be set first (gpu/poollayerbuilder.h)
    p.shape(8, 7, 5, 8).global_pool()
    assert p.downsample_ == [5, 7] and p.poolsize_ == [5, 7]
    c = fa.ConcatLayerBuilder("cat").input(23, 0).input(52, 0)
    assert c.inputChannels_ == 75


def test_layer_types_keep_reference_numbers():
    # fyusenet/base/layerflags.h:125-160
    assert (fa.LayerType.ADD, fa.LayerType.CONVOLUTION2D, fa.LayerType.TRANSCONVOLUTION2D, fa.LayerType.MAXPOOL2D) == (1, 6, 8, 10)
    assert (fa.LayerType.DOWNLOAD, fa.LayerType.UPLOAD, fa.LayerType.BATCHNORM, fa.LayerType.GEMM, fa.LayerType.CUSTOM) == (26, 27, 30, 31, 32)


def test_factory_rejects_duplicates_and_bad_numbers():
    class Dummy:
        _h = None
    f = fa.LayerFactory(Dummy())
    fa.ConvLayerBuilder(3, "a").type(fa.LayerType.CONVOLUTION2D).number(1).push(f)
    with pytest.raises(fa.FynException) as e:
        fa.ConvLayerBuilder(3, "b").type(fa.LayerType.CONVOLUTION2D).number(1).push(f)
    assert e.value.code == capi.ERR_DUPLICATE and "already taken" in str(e.value)
    with pytest.raises(fa.FynException):
        f.pushBuilder(fa.ConvLayerBuilder(3, "c").type(fa.LayerType.CONVOLUTION2D))  # number -1


def test_no_gpu_fails_loudly():
    if os.path.exists("/dev/kfd"):
        pytest.skip("GPU present")
    h = ctypes.c_void_p()
    rc = capi.lib().fyn_net_create(0, 0, ctypes.byref(h))
    assert rc == capi.ERR_DEVICE and b"hip" in capi.lib().fyn_last_error().lower()


def test_bench_refuses_more_than_one_gpu():
    """The engine runs on one GPU; bench.py says so instead of pretending to scale."""
    import subprocess, sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)
    assert not r.stdout.strip().startswith("{")   # (no record is printed)


def test_prng_is_stable():
    # golden values pin the generator so that every machine sees the same tensors
    from fyusenet_amd import prng
    u = prng.uniform(1234, (4,), -1, 1)
    n = prng.normal(99, (3,))
    assert u.dtype.name == "float32" and n.dtype.name == "float32"
    assert list(map(float, prng.uniform(1234, (4,), -1, 1))) == list(map(float, u))
    assert abs(float(prng.normal(5, (200000,)).std()) - 1.0) < 0.01
    assert abs(float(prng.uniform(6, (200000,), 0, 1).mean()) - 0.5) < 0.01


def test_resnet50_sample_weight_layout_matches_the_reference_file_layout():
    """Byte offsets derived from the layer descriptions against the values the reference hard-codes
    (samples/samplenetworks/resnet50.cpp:539-677); none of this needs the library."""
    from fyusenet_amd import samples

    class _Dry(samples.ResNet50Sample):
        def __init__(self):   # graph description only, no engine handle
            self._weights, self._specs, self._edges, self._file_order = None, [], [], []
            self._define()

        def __del__(self):
            pass

    net = _Dry()
    lay = net.weight_layout()
    assert net.total_weight_bytes() == samples.RESNET50_TOTAL_WEIGHT_BYTES == 102304184
    anchors = {2: (0, 24), 3: (24, 38400), 5: (38424, 512), 6: (38936, 17152), 8: (56088, 148224), 9: (204312, 66560),
               7: (270872, 66560), 10: (337432, 2048), 17: (837144, 68608), 19: (1893912, 526336), 20: (1038360, 591360),
               35: (9736728, 2101248), 36: (6321688, 2362368), 57: (33159704, 1060864), 59: (49969688, 8396800),
               62: (58366488, 16384), 69: (89889304, 4218880), 72: (94108184, 8196000)}
    for no, v in anchors.items():
        assert lay[no] == v, (no, lay[no], v)
    assert len(lay) == 68 and len(net._specs) == 72 and len(net._edges) == 87
    # every edge joins layers whose shapes agree
    spec = {no: b for no, b, _ in net._specs}
    for src, dst, port in net._edges:
        s, d = spec[src], spec[dst]
        if port == 0:
            assert s.outputChannels_ == d.inputChannels_, (src, dst)


def test_style_net_sample_weight_offsets_match_the_reference_tables():
    """Float offsets derived from the layer descriptions against the tables the reference hard-codes
    (samples/samplenetworks/stylenet3x3.cpp:41-50, stylenet9x9.cpp:41-56) and its stream sizes (stylenet3x3.h:53,
    stylenet9x9.h:59); none of this needs the library."""
    from fyusenet_amd import samples

    class _Dry(samples.StyleNetSample):
        def __init__(self, kernel):   # graph description only, no engine handle
            self.kernel, self.width, self.height, self.blocks = kernel, 64, 48, 2 if kernel == 3 else 5
            self.DECONV1 = self.FIRST_RES + 2 * self.blocks
            self.DECONV2, self.DECONV3, self.SIGMOID, self.DOWNLOAD = (self.DECONV1 + i for i in (1, 2, 3, 4))
            self._weights, self._specs, self._edges, self._file_order = None, [], [], []
            self._define()

        def __del__(self):
            pass

    n3 = _Dry(3)
    # enum of stylenet3x3.h:39-51: CONV1 1, CONV2 2, CONV3 3, RES1_1..RES2_2 4..7, DECONV1..3 8..10, SIGMOID 11, DOWNLOAD 12
    assert n3.weight_offsets() == {1: 0, 2: 336, 3: 2516, 4: 19475, 5: 33915, 6: 48355, 7: 62795, 8: 9756, 9: 16976, 10: 19148}
    assert n3.total_weight_bytes() == 4 * samples.STYLENET3X3_WEIGHT_FLOATS == 4 * 77235
    assert (n3.SIGMOID, n3.DOWNLOAD) == (11, 12) and len(n3._edges) == 14
    n9 = _Dry(9)
    assert n9.weight_offsets() == {1: 0, 2: 2928, 3: 5108, 4: 24659, 5: 39099, 6: 53539, 7: 67979, 8: 82419, 9: 96859, 10: 111299,
                                   11: 125739, 12: 140179, 13: 154619, 14: 12348, 15: 19568, 16: 21740}
    assert n9.total_weight_bytes() == 4 * samples.STYLENET9X9_WEIGHT_FLOATS == 4 * 169059
    assert (n9.SIGMOID, n9.DOWNLOAD) == (17, 18) and len(n9._edges) == 23
    spec = {no: b for no, b, _ in n9._specs}
    assert spec[n9.DECONV2].sourceStep_ == 0.25 and spec[n9.DECONV2].downsample_[0] == 2 and spec[n9.DECONV3].kernel_ == 9
