"""A residual block's 1x1 shortcut projection computed by the 1x1 layer that adds it: one reduction over two tensors
(the layer's own input and the projection's), the projection's tensor never written.  Parity against the oracle,
agreement with the two launches, and the conditions under which the engine keeps the layers apart.  Tolerances: rel-L2
<= 1e-4 (fp32 storage), <= 2e-3 (fp16 storage)."""
import numpy as np
import pytest

import fyusenet_amd as fa
from fyusenet_amd import networks, prng
from fyusenet_amd.builders import ActType, UpDownLayerBuilder
from oracle import oracle as O
from util import combos, rel_l2

pytestmark = pytest.mark.gpu
TOL = {fa.STORAGE_F32: 1e-4, fa.STORAGE_F16: 2e-3}


class Bottleneck(networks._StreamNet):
    """upload -> 1x1 front -> [1x1 projection (step s)] and [1x1 reduce -> 3x3 (step s) -> 1x1 expand + projection] ->
    download: the first block of a ResNet stage (samples/samplenetworks/resnet50.cpp:260-275)."""
    config_id = 3

    def __init__(self, storage, cin, mid, cout, h, w, stride, res_act=ActType.NONE, second_reader=False, res_bn=False, scale_decades=0):
        super().__init__(storage)
        self.res_bn = res_bn
        self.scale_decades = scale_decades
        self.cin, self.mid, self.cout, self.h, self.w, self.stride = cin, mid, cout, h, w, stride
        self.res_act, self.second_reader = res_act, second_reader

    def define(self):
        R = ActType.RELU
        ho, wo = self.h // self.stride, self.w // self.stride
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.UPLOAD, "upload").number(0).shape(self.cin, self.h, self.w, self.cin))
        self.conv(1, "front", 1, self.cin, self.cin, self.h, self.w, 0)
        self.conv(2, "projection", 1, self.cin, self.cout, self.h, self.w, 1, stride=self.stride, act=R)
        self.conv(3, "reduce", 1, self.cin, self.mid, self.h, self.w, 1, act=R, pad_out=1)
        self.conv(4, "spatial", 3, self.mid, self.mid, self.h, self.w, 3, stride=self.stride, act=R)
        self.conv(5, "expand", 1, self.mid, self.cout, ho, wo, 4, act=R, residual=2, res_act=self.res_act)
        if self.res_bn:   # the layer's batch-norm scale multiplies what it adds as well (ConvLayerBuilder::residual(act, true))
            self._builders[-1].residual(self.res_act, True)
        if self.scale_decades:   # batch-norm scales of the projection and of the adding layer log-uniform over so many decades
            for idx, (no, gen) in enumerate(self._blocks):
                if no in (2, 5):
                    self._blocks[idx] = (no, lambda g=gen, n=no: self._spread(g(), n))
        last = 5
        if self.second_reader:   # something else reads the projection's tensor
            self.conv(6, "side", 1, self.cout, 32, ho, wo, 2, act=R)
            last = 6
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.DOWNLOAD, "download").number(last + 1).shape(self.cout, ho, wo, self.cout).deep())
        self._edges.append((5, last + 1, 0))
        self.output_layer = last + 1

    def _spread(self, blk, no):
        # (downwards from 1, so that fp16 tensors hold the results)
        blk[-2 * self.cout:-self.cout] = (10.0 ** prng.uniform(8101 + no, (self.cout,), -float(self.scale_decades), 0.0)).astype(np.float32)
        return blk

    def makeInput(self):
        return prng.uniform(1709 + self.cin + self.h, (self.cin, self.h, self.w), -1.0, 1.0)

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


CASES = [
    # (cin, mid, cout, h, w, step)
    (64, 64, 256, 28, 28, 1),        # stage 1 of ResNet-50 (smaller): 2 + 2 chunks
    (256, 128, 512, 28, 28, 2),      # stage 2: the projection reads every other pixel; 4 + 8 chunks
    (512, 256, 1024, 14, 14, 2),     # stage 3: 8 + 16 chunks
    (1024, 512, 2048, 14, 14, 2),    # stage 4: 16 + 32 chunks
    (96, 48, 80, 13, 11, 1),         # channel counts that are no multiples of 32 or of the block, ragged tiles; 2 + 3 chunks rounded up to 8
    (40, 24, 72, 9, 15, 2),          # odd sizes with step 2
]


@pytest.mark.parametrize(*combos(
    # (the residual's batch-norm is varied on the smaller cases)
    lambda case, res_bn, storage: not (res_bn and case[0] > 256),
    case=(CASES, lambda c: "%d_%d_%d_%dx%d_s%d" % c), res_bn=([False, True], lambda r: "bn_on_residual" if r else "plain"),
    storage=([fa.STORAGE_F32, fa.STORAGE_F16], lambda st: "f32" if st == fa.STORAGE_F32 else "f16")))
def test_projection_inside_the_layer_that_adds_it(case, res_bn, storage, monkeypatch):
    cin, mid, cout, h, w, stride = case
    monkeypatch.setenv("FYNHIP_FORCE_PROJECTION_FUSION", "1")
    net = Bottleneck(storage, cin, mid, cout, h, w, stride, res_bn=res_bn)
    x, got, infos = run(net)
    desc = net.describe()
    net.cleanup()
    print("  ", infos["projection"][:100], "|", infos["expand"][:170], flush=True)
    assert "launch of layer 5" in infos["projection"] and "over two tensors" in infos["expand"] and "projection 2" in infos["expand"]
    ref = O.run_network(desc, {net.input_key: x})[net.output_layer]
    err = rel_l2(got, ref)
    print("   rel_l2=%.3e" % err, flush=True)
    assert err <= TOL[storage]
    monkeypatch.delenv("FYNHIP_FORCE_PROJECTION_FUSION")
    monkeypatch.setenv("FYNHIP_NO_PROJECTION_FUSION", "1")
    twin = Bottleneck(storage, cin, mid, cout, h, w, stride, res_bn=res_bn)
    _, two, infos2 = run(twin)
    twin.cleanup()
    assert "no launch of its own" not in infos2["projection"]
    # (the folded scales multiply the weights before their fp16 split instead of the sum behind it, and the projection's
    # result is not rounded to the storage type on its way into the sum: agreement, not equality)
    assert rel_l2(got, two) <= (5e-6 if storage == fa.STORAGE_F32 else 1.5e-3)


@pytest.mark.parametrize("why", ["relu_on_residual", "second_reader", "no_reuse"])
def test_projection_keeps_its_launch_when_it_has_to(why, monkeypatch):
    """An activation between the projection and the sum, another reader of the projection's tensor, or a network set up
    without buffer reuse (every tensor readable afterwards): two launches."""
    monkeypatch.setenv("FYNHIP_FORCE_PROJECTION_FUSION", "1")
    net = Bottleneck(fa.STORAGE_F32, 256, 128, 512, 14, 14, 1, res_act=ActType.RELU if why == "relu_on_residual" else ActType.NONE,
                     second_reader=(why == "second_reader"))
    x, got, infos = run(net, reuse=(why != "no_reuse"))
    desc = net.describe()
    net.cleanup()
    assert "no launch of its own" not in infos["projection"] and "two tensors" not in infos["expand"]
    ref = O.run_network(desc, {net.input_key: x})[net.output_layer]
    assert rel_l2(got, ref) <= TOL[fa.STORAGE_F32]


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("decades", [4, 8])
def test_projection_with_scales_of_very_different_magnitude(decades, storage, monkeypatch):
    """The one launch carries both layers' batch-norm scales on its weight rows, under one common power of two.  Scales
    spread over four decades keep the bound; over eight decades (beyond the 2^16 between rows that the packing allows)
    the pair runs as two launches, each layer's scale on its fp32 sum, and keeps it as well."""
    monkeypatch.setenv("FYNHIP_FORCE_PROJECTION_FUSION", "1")
    net = Bottleneck(storage, 64, 64, 256, 28, 28, 1, scale_decades=decades)
    x, got, infos = run(net)
    desc = net.describe()
    net.cleanup()
    print("  ", infos["projection"][:100], "|", infos["expand"][:120], flush=True)
    if decades <= 4:
        assert "launch of layer 5" in infos["projection"] and "over two tensors" in infos["expand"]
    else:
        assert "no launch of its own" not in infos["projection"] and "two tensors" not in infos["expand"]
    ref = O.run_network(desc, {net.input_key: x})[net.output_layer]
    err = rel_l2(got, ref)
    print("   rel_l2=%.3e" % err, flush=True)
    assert err <= TOL[storage]
