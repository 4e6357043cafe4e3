"""A depthwise 3x3 layer that runs inside the launch of a neighbour: of the 1x1 layer in front of it (the first half of
an inverted-residual block as one launch; the expanded tensor is never written) or, in the staging, of the 1x1 layer
behind it (the second half; the depthwise layer's tensor is never written).  Parity against the oracle, equality with
the two-launch form, and the conditions under which the engine leaves the layers apart.  Tolerances: rel-L2 <= 1e-4
(fp32 storage), <= 2e-3 (fp16 storage)."""
import numpy as np
import pytest

import fyusenet_amd as fa
from fyusenet_amd import networks, prng
from fyusenet_amd.builders import ActType, UpDownLayerBuilder
from oracle import oracle as O
from util import combos, rel_l2

pytestmark = pytest.mark.gpu
TOL = {fa.STORAGE_F32: 1e-4, fa.STORAGE_F16: 2e-3}


class Block(networks._StreamNet):
    """upload -> 1x1 expand -> depthwise 3x3 (step 1 or 2, clip on fetch) -> 1x1 project (clip on fetch, optional residual
    from the block's input) -> download."""
    config_id = 4

    def __init__(self, storage, cin, exp, cout, h, w, stride, residual, side_reader=False, expand_side_reader=False):
        super().__init__(storage)
        self.cin, self.exp, self.cout, self.h, self.w, self.stride, self.residual, self.side_reader = cin, exp, cout, h, w, stride, residual, side_reader
        self.expand_side_reader = expand_side_reader

    def define(self):
        C, c6 = ActType.CLIP, (0.0, 6.0)
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.UPLOAD, "upload").number(0).shape(self.cin, self.h, self.w, self.cin))
        self.conv(1, "expand", 1, self.cin, self.exp, self.h, self.w, 0, pad_out=1)
        self.conv(2, "dw", 3, self.exp, self.exp, self.h, self.w, 1, stride=self.stride, act=C, clip=c6, groups=self.exp)
        ho, wo = self.h // self.stride, self.w // self.stride
        self.conv(3, "project", 1, self.exp, self.cout, ho, wo, 2, act=C, clip=c6, residual=0 if self.residual else None)
        last = 3
        if self.side_reader:   # a second reader of the depthwise layer's tensor
            self.conv(4, "side", 1, self.exp, 16, ho, wo, 2, act=C, clip=c6)
            last = 4
        if self.expand_side_reader:   # a second reader of the expanded tensor (which has a halo of 1)
            self.conv(4, "side", 3, self.exp, 16, self.h, self.w, 1, act=C, clip=c6)
            last = 4
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.DOWNLOAD, "download").number(last + 1).shape(self.cout, ho, wo, self.cout).deep())
        self._edges.append((3, last + 1, 0))
        self.output_layer = last + 1

    def makeInput(self):
        return prng.uniform(977 + self.cin + self.h, (self.cin, self.h, self.w), -1.0, 1.0)

    def setInput(self, x):
        self.layers[0].setInput(x, 0)

    input_key = (0, 0)


def run(net, reuse=True):
    net.setup(reuseBuffers=reuse)
    x = net.makeInput()
    net.setInput(x)
    net.forward()
    net.finish()
    out = net.getOutput(net.output_layer)
    infos = {lyr.name: lyr.kernelInfo() for lyr in net.layers}
    return x, out, infos


def assert_same_as_two_launches(fused, two, storage):
    """fp32 storage: the same bits (same arithmetic in the same order).  fp16 storage: the depthwise layer's value is
    rounded to fp16 on its way to the 1x1 layer in both forms, but the compiler may fold that rounding into the
    multiply-add in front of it in one kernel and not in the other (one rounding instead of two): a few values per
    thousand differ in their last bit, and a few outputs with them."""
    if storage == fa.STORAGE_F32:
        assert np.array_equal(fused, two)
        return
    d = np.abs(fused.astype(np.float64) - two.astype(np.float64))
    assert (d > 0).mean() <= 0.02, "differing outputs: %d of %d" % ((d > 0).sum(), d.size)
    assert d.max() <= 2.0 ** -9 * np.abs(two).max()


CASES = [
    # (cin, expanded channels, cout, h, w, step, residual)
    (16, 96, 24, 28, 28, 1, False),      # one chunk per wave (96 channels padded to 128)
    (24, 144, 24, 20, 24, 1, True),      # two chunks per wave, residual add in the pointwise epilogue
    (32, 192, 64, 14, 14, 2, False),     # step 2
    (64, 384, 96, 14, 14, 1, False),     # three chunks per wave, three blocks of 32 output channels
    (64, 384, 64, 14, 14, 2, False),     # three chunks per wave, step 2: texels in two rounds
    (80, 480, 112, 7, 7, 1, False),      # 15 chunks in use of 16
    (32, 32, 16, 26, 22, 1, False),      # a single chunk in use, ragged tiles
    (24, 144, 40, 13, 11, 2, False),     # odd input size with step 2, 40 output channels (last block partly empty)
]


FRONT_CASES = CASES + [
    (160, 960, 320, 7, 7, 1, False),     # five chunks of input channels, 15 blocks of expanded channels
    (96, 576, 160, 14, 14, 2, False),
    (16, 96, 24, 112, 112, 2, False),    # the largest resolution of the stack
]


@pytest.mark.parametrize(*combos(
    # (the 16-channel blocks are for layers with few tiles)
    lambda narrow, case, storage: not (narrow and case[3] * case[4] > 60 * 60),
    narrow=([0, 1], lambda n: "blocks16" if n else "blocks64"),
    case=(FRONT_CASES, lambda c: "%dto%dto%d_%dx%d_s%d%s" % (c[0], c[1], c[2], c[3], c[4], c[5], "_res" if c[6] else "")),
    storage=([fa.STORAGE_F32, fa.STORAGE_F16], lambda st: "f32" if st == fa.STORAGE_F32 else "f16")))
def test_depthwise_inside_the_launch_of_the_expand_layer(narrow, case, storage, monkeypatch):
    cin, exp, cout, h, w, stride, residual = case
    monkeypatch.setenv("FYNHIP_FORCE_DW_FUSION", "1")
    monkeypatch.setenv("FYNHIP_EDW_NARROW", str(narrow))
    net = Block(storage, cin, exp, cout, h, w, stride, residual)
    x, got, infos = run(net)
    desc = net.describe()
    net.cleanup()
    print("  ", infos["dw"], "|", infos["expand"][:120], flush=True)
    assert "launch of layer 1" in infos["dw"] and "conv_e16dw" in infos["expand"] and "depthwise 3x3 layer 2" in infos["expand"]
    assert ("and 16 expanded channels" if narrow else "and 64 expanded channels") in infos["expand"]
    ref = O.run_network(desc, {net.input_key: x})[net.output_layer]
    err = rel_l2(got, ref)
    print("   rel_l2=%.3e" % err, flush=True)
    assert err <= TOL[storage]
    monkeypatch.setenv("FYNHIP_NO_DW_FUSION", "1")
    twin = Block(storage, cin, exp, cout, h, w, stride, residual)
    _, two, infos2 = run(twin)
    twin.cleanup()
    assert infos2["dw"] == "dwconv3x3"
    # (the 1x1 layer on its own may run a kernel that sums the reduction in another order: no bit-equality here)
    assert rel_l2(got, two) <= (2e-6 if storage == fa.STORAGE_F32 else 1e-3)


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: "%dto%dto%d_%dx%d_s%d%s" % (c[0], c[1], c[2], c[3], c[4], c[5], "_res" if c[6] else ""))
def test_depthwise_inside_pointwise_staging(case, storage, monkeypatch):
    cin, exp, cout, h, w, stride, residual = case
    monkeypatch.setenv("FYNHIP_FORCE_KR16_CONV", "1")
    monkeypatch.setenv("FYNHIP_FORCE_DW_FUSION", "1")
    monkeypatch.setenv("FYNHIP_NO_EDW_FUSION", "1")
    net = Block(storage, cin, exp, cout, h, w, stride, residual)
    x, got, infos = run(net)
    desc = net.describe()
    net.cleanup()
    print("  ", infos["dw"], "|", infos["project"], flush=True)
    assert "launch of layer 3" in infos["dw"] and "depthwise 3x3 layer 2" in infos["project"]
    ref = O.run_network(desc, {net.input_key: x})[net.output_layer]
    err = rel_l2(got, ref)
    print("   rel_l2=%.3e" % err, flush=True)
    assert err <= TOL[storage]
    monkeypatch.setenv("FYNHIP_NO_DW_FUSION", "1")
    twin = Block(storage, cin, exp, cout, h, w, stride, residual)
    _, two, infos2 = run(twin)
    twin.cleanup()
    assert infos2["dw"] == "dwconv3x3"
    assert_same_as_two_launches(got, two, storage)


D16_CASES = [
    (16, 32, 16, 40, 40, 1, False),      # one chunk, one fragment of output channels
    (16, 96, 24, 36, 36, 2, False),      # three chunks, step 2
    (24, 48, 24, 30, 34, 1, True),       # a chunk and a half, residual add
    (32, 64, 80, 20, 20, 1, False),      # five fragments: more than one per wave, one ahead of their use
]


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("case", D16_CASES, ids=lambda c: "%dto%dto%d_%dx%d_s%d%s" % (c[0], c[1], c[2], c[3], c[4], c[5], "_res" if c[6] else ""))
def test_depthwise_inside_the_lds_free_pointwise_kernel(case, storage, monkeypatch):
    """The same second half of the block where the 1x1 layer runs the LDS-free kernel (many positions, up to 96
    channels): every wave computes the depthwise layer for its positions."""
    cin, exp, cout, h, w, stride, residual = case
    monkeypatch.setenv("FYNHIP_FORCE_D16_CONV", "1")
    monkeypatch.setenv("FYNHIP_FORCE_DW_FUSION", "1")
    monkeypatch.setenv("FYNHIP_NO_EDW_FUSION", "1")
    net = Block(storage, cin, exp, cout, h, w, stride, residual)
    x, got, infos = run(net)
    desc = net.describe()
    net.cleanup()
    print("  ", infos["dw"], "|", infos["project"], flush=True)
    assert "launch of layer 3" in infos["dw"] and "conv_d16" in infos["project"] and "depthwise 3x3 layer 2" in infos["project"]
    ref = O.run_network(desc, {net.input_key: x})[net.output_layer]
    err = rel_l2(got, ref)
    print("   rel_l2=%.3e" % err, flush=True)
    assert err <= TOL[storage]
    monkeypatch.setenv("FYNHIP_NO_DW_FUSION", "1")
    twin = Block(storage, cin, exp, cout, h, w, stride, residual)
    _, two, infos2 = run(twin)
    twin.cleanup()
    assert infos2["dw"] == "dwconv3x3"
    assert_same_as_two_launches(got, two, storage)


def test_layers_stay_apart_when_the_tensor_is_needed(monkeypatch):
    """No fusion when the tensor between the two layers has a second reader, or when the caller keeps every layer's
    tensor (buffer reuse off); per-layer timing runs the layers apart and leaves the results unchanged."""
    monkeypatch.setenv("FYNHIP_FORCE_KR16_CONV", "1")
    monkeypatch.setenv("FYNHIP_FORCE_DW_FUSION", "1")
    # a second reader of the depthwise layer's tensor: the 1x1 layer behind it must fetch it; the layer in front may still run it
    net = Block(fa.STORAGE_F16, 16, 96, 24, 28, 28, 1, False, side_reader=True)
    _, _, infos = run(net)
    net.cleanup()
    assert "launch of layer 1" in infos["dw"]
    monkeypatch.setenv("FYNHIP_NO_EDW_FUSION", "1")
    net = Block(fa.STORAGE_F16, 16, 96, 24, 28, 28, 1, False, side_reader=True)
    _, _, infos = run(net)
    net.cleanup()
    assert infos["dw"] == "dwconv3x3"
    net = Block(fa.STORAGE_F16, 96, 576, 160, 14, 14, 1, False)   # (more than 512 channels: no variant of the staging form)
    _, _, infos = run(net)
    net.cleanup()
    assert infos["dw"] == "dwconv3x3"
    monkeypatch.delenv("FYNHIP_NO_EDW_FUSION")
    # a second reader of the expanded tensor
    net = Block(fa.STORAGE_F16, 16, 96, 24, 28, 28, 1, False, expand_side_reader=True)
    _, _, infos = run(net)
    net.cleanup()
    assert "conv_e16dw" not in infos["expand"] and "launch of layer 3" in infos["dw"]
    net = Block(fa.STORAGE_F16, 16, 96, 24, 28, 28, 1, False)
    _, _, infos = run(net, reuse=False)
    dw_out = net.layers[2].copyResult()
    ex_out = net.layers[1].copyResult()
    net.cleanup()
    assert infos["dw"] == "dwconv3x3" and np.abs(dw_out).max() > 0 and np.abs(ex_out).max() > 0
    for no_edw in (False, True):
        if no_edw:
            monkeypatch.setenv("FYNHIP_NO_EDW_FUSION", "1")
        net = Block(fa.STORAGE_F16, 16, 96, 24, 28, 28, 1, False)
        _, fused, infos = run(net)
        assert "inside the launch" in infos["dw"]
        net.enableTimings(True)
        net.forward()
        net.finish()
        apart = net.getOutput(net.output_layer)
        net.enableTimings(False)
        net.forward()
        net.finish()
        again = net.getOutput(net.output_layer)
        net.cleanup()
        assert rel_l2(fused, apart) <= 1e-3
        assert np.array_equal(fused, again)


class Chain(networks._StreamNet):
    """upload -> depthwise 3x3 -> 1x1 -> depthwise 3x3 -> 1x1 -> download (the MobileNetV1 pattern): the middle 1x1
    layer has a depthwise layer on either side and can run only one of them inside its launch."""
    config_id = 4

    def __init__(self, storage, c, e, cout, h, w):
        super().__init__(storage)
        self.c, self.e, self.cout, self.h, self.w = c, e, cout, h, w

    def define(self):
        C, c6 = ActType.CLIP, (0.0, 6.0)
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.UPLOAD, "upload").number(0).shape(self.c, self.h, self.w, self.c).outputPadding(1))
        self.conv(1, "dw1", 3, self.c, self.c, self.h, self.w, 0, groups=self.c)
        self.conv(2, "pw1", 1, self.c, self.e, self.h, self.w, 1, act=C, clip=c6, pad_out=1)
        self.conv(3, "dw2", 3, self.e, self.e, self.h, self.w, 2, act=C, clip=c6, groups=self.e)
        self.conv(4, "pw2", 1, self.e, self.cout, self.h, self.w, 3, act=C, clip=c6)
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.DOWNLOAD, "download").number(5).shape(self.cout, self.h, self.w, self.cout).deep())
        self._edges.append((4, 5, 0))
        self.output_layer = 5

    def makeInput(self):
        return prng.uniform(4211 + self.c + self.h, (self.c, self.h, self.w), -1.0, 1.0)

    def setInput(self, x):
        self.layers[0].setInput(x, 0)

    input_key = (0, 0)


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("form", ["kr16", "d16"])
def test_pointwise_layer_between_two_depthwise_layers_takes_one(storage, form, monkeypatch):
    """The 1x1 layer in the middle is a candidate for both passes (the depthwise layer behind it as one launch, the one
    in front of it inside its staging); it may take one, and every depthwise layer is computed exactly once."""
    monkeypatch.setenv("FYNHIP_FORCE_KR16_CONV" if form == "kr16" else "FYNHIP_FORCE_D16_CONV", "1")
    monkeypatch.setenv("FYNHIP_FORCE_DW_FUSION", "1")
    net = Chain(storage, 32, 64, 48, 28, 28)
    x, got, infos = run(net)
    desc = net.describe()
    net.cleanup()
    print("  ", {k: v[:90] for k, v in infos.items() if k != "upload"}, flush=True)
    assert "conv_e16dw" in infos["pw1"] and "launch of layer 2" in infos["dw2"]
    assert infos["dw1"] == "dwconv3x3", "the layer that already runs the depthwise layer behind it must fetch the one in front of it"
    ref = O.run_network(desc, {net.input_key: x})[net.output_layer]
    err = rel_l2(got, ref)
    print("   rel_l2=%.3e" % err, flush=True)
    assert err <= TOL[storage]


class Interleaved(networks._StreamNet):
    """Two graphs in which a layer numbered between the fused pair lives in the buffer that the fused launch would read
    late or write early.
    kind "late" (depthwise -> 1x1): 1 a (1x1, halo) -> 2 dw -> 4 pw, and 3 mid (1x1 from the upload, same geometry as a's
        tensor, which is free behind layer 2): a launch of layer 4 that computes layer 2 itself would read a's buffer
        after layer 3 has overwritten it.
    kind "early" (1x1 -> depthwise): 1 pre -> 3 side, 2 expand -> 4 dw -> 5 project; the depthwise layer's output takes
        pre's buffer (free behind layer 3): a launch of layer 2 that also runs layer 4 would write into it before layer
        3 has read it."""
    config_id = 4

    def __init__(self, storage, kind, c=32, h=20, w=24):
        super().__init__(storage)
        self.kind, self.c, self.h, self.w = kind, c, h, w

    def define(self):
        C, c6 = ActType.CLIP, (0.0, 6.0)
        c, h, w = self.c, self.h, self.w
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.UPLOAD, "upload").number(0).shape(c, h, w, c))
        if self.kind == "late":
            self.conv(1, "a", 1, c, c, h, w, 0, pad_out=1)
            self.conv(2, "dw", 3, c, c, h, w, 1, act=C, clip=c6, groups=c)
            self.conv(3, "mid", 1, c, c, h, w, 0, pad_out=1)
            self.conv(4, "pw", 1, c, 48, h, w, 2, act=C, clip=c6)
            self.conv(5, "tail", 3, c, 16, h, w, 3, act=C, clip=c6)
            self.outputs = (4, 5)
        else:
            self.conv(1, "pre", 1, c, c, h, w, 0)
            self.conv(2, "expand", 1, c, c, h, w, 0, pad_out=1)
            self.conv(3, "side", 1, c, 16, h, w, 1, act=C, clip=c6)
            self.conv(4, "dw", 3, c, c, h, w, 2, act=C, clip=c6, groups=c)
            self.conv(5, "project", 1, c, 48, h, w, 4, act=C, clip=c6)
            self.outputs = (3, 5)

    def makeInput(self):
        return prng.uniform(5003 + self.c + self.h, (self.c, self.h, self.w), -1.0, 1.0)

    def setInput(self, x):
        self.layers[0].setInput(x, 0)

    input_key = (0, 0)


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("kind", ["late", "early"])
def test_no_fusion_across_a_layer_that_reuses_the_buffer(kind, storage, monkeypatch):
    monkeypatch.setenv("FYNHIP_FORCE_KR16_CONV", "1")
    monkeypatch.setenv("FYNHIP_FORCE_DW_FUSION", "1")
    if kind == "late":
        monkeypatch.setenv("FYNHIP_NO_EDW_FUSION", "1")
    net = Interleaved(storage, kind)
    net.setup(reuseBuffers=True)
    x = net.makeInput()
    net.setInput(x)
    net.forward()
    net.finish()
    got = {no: net.layers[no].copyResult() for no in net.outputs}
    infos = {lyr.name: lyr.kernelInfo() for lyr in net.layers}
    desc = net.describe()
    net.cleanup()
    print("  ", {k: v[:80] for k, v in infos.items() if k != "upload"}, flush=True)
    if kind == "late":
        assert infos["dw"] == "dwconv3x3"
    else:
        assert "conv_e16dw" not in infos["expand"]
    ref = O.run_network(desc, {net.input_key: x})
    for no in net.outputs:
        err = rel_l2(got[no], ref[no])
        print("   layer %d rel_l2=%.3e" % (no, err), flush=True)
        assert err <= TOL[storage]


class TappedMobileNetV2(networks.MobileNetV2):
    """BASELINE's MobileNetV2-style graph with a download layer on the stem's and on every block's output: those tensors
    keep their buffers, so they can be read after a pass in which buffers are shared and the layers inside the blocks
    run fused (the taps are further readers of tensors between blocks, not of the tensors that the fusions remove)."""

    def define(self):
        super().define()
        taps = [b for b in self._builders if b.name_ == "stem" or b.name_.endswith("_project")]
        for i, b in enumerate(taps):
            c, h, w = b.outputChannels_, b.height_ // b.downsample_[1], b.width_ // b.downsample_[0]
            self._add(UpDownLayerBuilder(UpDownLayerBuilder.DOWNLOAD, "tap_" + b.name_).number(1000 + i).shape(c, h, w, c).inputPadding(b.outputPadding_).deep())
            self._edges.append((b.number_, 1000 + i, 0))


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
def test_config4_fused_blocks_one_by_one_on_the_engines_own_inputs(storage, monkeypatch):
    """Every inverted-residual block of the fused stack against the oracle evaluated on the engine's own block input
    (and residual): the per-layer bound (1e-4 / 2e-3) on each block, in the storage type the benchmark runs, instead of
    only the end-to-end bound of two free-running fp16 chains."""
    monkeypatch.setenv("FYNHIP_FORCE_DW_FUSION", "1")
    net = TappedMobileNetV2(storage)
    x, got, infos = run(net)
    desc = net.describe()
    number = {lyr.name: lyr.number for lyr in net.layers}
    fused = [n for n, i in infos.items() if "inside the launch" in i]
    assert len(fused) >= 8
    prev = number["stem"]
    tensors = {prev: net.layers[prev].copyResult()}
    worst = 0.0
    for i in range(len(networks.MobileNetV2.BLOCKS)):
        part = [number[n] for n in ("b%d_expand" % i, "b%d_dw" % i, "b%d_project" % i) if n in number]
        out_no = number["b%d_project" % i]
        tensors[out_no] = net.layers[out_no].copyResult()
        ref = O.run_network(desc, {}, known={prev: tensors[prev]}, only=set(part))[out_no]
        err = rel_l2(tensors[out_no], ref)
        worst = max(worst, err)
        print("   block %2d (%s) rel_l2=%.3e" % (i, "fused" if "b%d_dw" % i in fused else "apart", err), flush=True)
        assert err <= TOL[storage], "block %d" % i
        prev = out_no
    net.cleanup()


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
def test_config4_mobilenetv2_with_fused_blocks(storage, monkeypatch):
    """The whole MobileNetV2-style graph with every eligible depthwise layer fused, eager and as a replayed graph,
    against the same graph with the layers apart and against the oracle's free-running chain."""
    monkeypatch.setenv("FYNHIP_FORCE_DW_FUSION", "1")
    net = networks.MobileNetV2(storage)
    x, got, infos = run(net)
    net.useGraph(True)
    net.forward()
    net.finish()
    net.forward()
    net.finish()
    replay = net.getOutput(net.output_layer)
    desc = net.describe()
    net.cleanup()
    fused = [n for n, i in infos.items() if "inside the launch" in i]
    print("   fused:", len(fused), fused, flush=True)
    assert len(fused) >= 8
    assert np.array_equal(got, replay)
    monkeypatch.setenv("FYNHIP_NO_DW_FUSION", "1")
    twin = networks.MobileNetV2(storage)
    _, two, _ = run(twin)
    twin.cleanup()
    # (last-bit differences of single values grow along the 52 layers of an untrained chain, fp16 storage most of all)
    assert rel_l2(got, two) <= (1e-4 if storage == fa.STORAGE_F32 else 5e-2)
    ref = O.run_network(desc, {net.input_key: x})[net.output_layer]
    assert rel_l2(got, ref) <= (1e-4 if storage == fa.STORAGE_F32 else 5e-2)
