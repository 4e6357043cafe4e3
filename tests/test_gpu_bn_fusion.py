"""A batch-norm layer (plain x * scale + bias between tensors of one geometry) that its readers apply themselves: the
convolution layers behind it stage from the batch-norm layer's input and apply scale and bias per channel before their
own activation; the layer's tensor is never written.  Parity against the oracle, equality with the separate launch, and
the conditions under which the engine leaves the layer alone.  Tolerances: rel-L2 <= 1e-4 (fp32 storage), <= 2e-3 (fp16
storage)."""
import numpy as np
import pytest

import fyusenet_amd as fa
from fyusenet_amd import networks, prng
from fyusenet_amd.builders import ActType, GPULayerBuilder, LayerType, UpDownLayerBuilder
from oracle import oracle as O
from util import rel_l2

pytestmark = pytest.mark.gpu
TOL = {fa.STORAGE_F32: 1e-4, fa.STORAGE_F16: 2e-3}


class PreActBlock(networks._StreamNet):
    """upload -> 1x1 conv -> batch-norm -> k x k conv with ReLU on fetch (-> a second reader) -> 1x1 conv with the
    residual from in front of the batch-norm layer -> download: the head of a pre-activation residual block as the
    reference's ResNet-50 sample graph spells it (samples/samplenetworks/resnet50.cpp:233-245)."""
    config_id = 3

    def __init__(self, storage, cin, mid, h, w, k=1, second_reader=False, bn_residual=False, download_bn=False):
        super().__init__(storage)
        self.cin, self.mid, self.h, self.w, self.k = cin, mid, h, w, k
        self.second_reader, self.bn_residual, self.download_bn = second_reader, bn_residual, download_bn

    def define(self):
        R = ActType.RELU
        pad = (self.k - 1) // 2
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.UPLOAD, "upload").number(0).shape(self.cin, self.h, self.w, self.cin))
        self.conv(1, "front", 1, self.cin, self.cin, self.h, self.w, 0, pad_out=pad)
        b = GPULayerBuilder("bn").type(LayerType.BATCHNORM).number(2).shape(self.cin, self.h, self.w, self.cin).deep()
        b.inputPadding(pad).outputPadding(pad)
        if self.bn_residual:
            b.residual(ActType.NONE)
            self._edges.append((1, 2, 1))
        seed = self._next_seed()
        c = self.cin
        self._add(b, lambda: np.concatenate([prng.uniform(seed, (c,), 0.5, 1.5), prng.normal(seed + 1, (c,), 0.0, 0.3)]).astype(np.float32))
        self._edges.append((1, 2, 0))
        self.conv(3, "reader", self.k, self.cin, self.mid, self.h, self.w, 2, act=R)
        last = 3
        if self.second_reader:
            self.conv(4, "reader2", 1, self.cin, 32, self.h, self.w, 2, act=R)
            last = 4
        self.conv(last + 1, "back", 1, self.mid, self.cin, self.h, self.w, 3, act=R, residual=1, res_pad=pad)
        out_src = 2 if self.download_bn else last + 1
        self._add(UpDownLayerBuilder(UpDownLayerBuilder.DOWNLOAD, "download").number(last + 2).shape(self.cin, self.h, self.w, self.cin).deep().inputPadding(pad if self.download_bn else 0))
        self._edges.append((out_src, last + 2, 0))
        self.output_layer = last + 2

    def makeInput(self):
        return prng.uniform(1301 + self.cin + self.h, (self.cin, self.h, self.w), -1.0, 1.0)

    def setInput(self, x):
        self.layers[0].setInput(x, 0)

    input_key = (0, 0)


def run(net):
    net.setup(reuseBuffers=True)
    x = net.makeInput()
    net.setInput(x)
    net.forward()
    net.finish()
    out = net.getOutput(net.output_layer)
    infos = {lyr.name: lyr.kernelInfo() for lyr in net.layers}
    return x, out, infos


CASES = [
    # (cin, mid, h, w, kernel of the reader, second reader)
    (256, 64, 14, 14, 1, False),     # the first layer of a ResNet stage-1 block, smaller
    (512, 128, 13, 9, 1, True),      # two readers, ragged tiles
    (1024, 256, 7, 7, 1, False),     # eight chunks per wave
    (96, 48, 9, 11, 1, False),       # channels that are no multiple of 128
    (2048, 64, 7, 7, 1, False),      # 64 chunks
]


D16_CASES = [
    (64, 64, 56, 56, 1, True),       # the first block of the reference's ResNet-50 graph: two readers behind the pooled tensor's batch-norm
    (96, 24, 37, 29, 1, False),      # three chunks, positions no multiple of 16
    (32, 144, 28, 28, 1, False),
]


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("form,case", [("kr16", c) for c in CASES] + [("d16", c) for c in D16_CASES],
                         ids=lambda v: v if isinstance(v, str) else "%dto%d_%dx%d_k%d%s" % (v[0], v[1], v[2], v[3], v[4], "_two" if v[5] else ""))
def test_batchnorm_applied_by_its_readers(form, case, storage, monkeypatch):
    cin, mid, h, w, k, two = case
    monkeypatch.setenv("FYNHIP_FORCE_KR16_CONV" if form == "kr16" else "FYNHIP_FORCE_D16_CONV", "1")
    net = PreActBlock(storage, cin, mid, h, w, k, second_reader=two)
    x, got, infos = run(net)
    desc = net.describe()
    net.cleanup()
    print("  ", infos["bn"], "|", infos["reader"], flush=True)
    assert "no launch of its own" in infos["bn"] and "batch-norm layer 2" in infos["reader"] and ("conv_" + form) in infos["reader"]
    if two:
        assert "batch-norm layer 2" in infos["reader2"]
    ref = O.run_network(desc, {net.input_key: x})[net.output_layer]
    err = rel_l2(got, ref)
    print("   rel_l2=%.3e" % err, flush=True)
    assert err <= TOL[storage]
    monkeypatch.setenv("FYNHIP_NO_BN_FUSION", "1")
    twin = PreActBlock(storage, cin, mid, h, w, k, second_reader=two)
    _, apart, infos2 = run(twin)
    twin.cleanup()
    assert infos2["bn"] == "batchnorm"
    # (the same arithmetic on the same values in both forms; fp16 storage: the batch-norm value is rounded to fp16 on
    # its way to the reader in both, but the compiler may fold that rounding into the multiply-add in one of them)
    if storage == fa.STORAGE_F32:
        assert np.array_equal(got, apart)
    else:
        assert rel_l2(got, apart) <= 1e-3


@pytest.mark.parametrize("why", ["bn_residual", "download_bn", "reader_not_resident", "no_reuse", "halo"])
def test_batchnorm_keeps_its_launch_when_it_has_to(why, monkeypatch):
    """A residual input on the batch-norm layer, a reader that is no convolution on the K-resident form, a network set up
    without buffer reuse (every tensor readable afterwards), or tensors with a halo (a 3x3 reader: the halo of the
    layer's output holds zeros, not the bias): the layer runs on its own."""
    if why != "reader_not_resident":
        monkeypatch.setenv("FYNHIP_FORCE_KR16_CONV", "1")
    else:
        monkeypatch.setenv("FYNHIP_NO_KR16_CONV", "1")
    net = PreActBlock(fa.STORAGE_F32, 256, 64, 14, 14, 3 if why == "halo" else 1, bn_residual=(why == "bn_residual"), download_bn=(why == "download_bn"))
    net.setup(reuseBuffers=(why != "no_reuse"))
    x = net.makeInput()
    net.setInput(x)
    net.forward()
    net.finish()
    got = net.getOutput(net.output_layer)
    infos = {lyr.name: lyr.kernelInfo() for lyr in net.layers}
    desc = net.describe()
    net.cleanup()
    assert infos["bn"] == "batchnorm" and "batch-norm" not in infos["reader"]
    ref = O.run_network(desc, {net.input_key: x})[net.output_layer]
    assert rel_l2(got, ref) <= TOL[fa.STORAGE_F32]


def test_reference_resnet50_sample_graph_with_batchnorm_layers_applied_by_their_readers(monkeypatch):
    """The reference's ResNet-50 sample graph set up for inference (buffer reuse on): the batch-norm layers in front of
    the blocks run inside the convolutions that read them; the logits against the oracle and against the same network
    with every layer launched on its own."""
    from fyusenet_amd import samples
    net = samples.ResNet50Sample(fa.STORAGE_F32)
    net.setup(reuseBuffers=True)
    x = net.makeInput()
    net.setInput(x)
    net.forward()
    net.finish()
    got = net.layers[net.GEMM].copyResult()
    infos = [lyr.kernelInfo() for lyr in net.layers]
    desc = net.describe()
    net.cleanup()
    gone = sum("no launch of its own" in i for i in infos)
    print("   batch-norm layers without a launch: %d of %d" % (gone, sum(i.startswith("batchnorm") for i in infos)), flush=True)
    assert gone >= 8   # (13 of 14 when every reader's timing picks the K-resident or the LDS-free form, as it does on the boxes seen)
    ref = O.run_network(desc, {net.input_key: x})[net.GEMM]
    assert rel_l2(got, ref) <= TOL[fa.STORAGE_F32]
    monkeypatch.setenv("FYNHIP_NO_BN_FUSION", "1")
    twin = samples.ResNet50Sample(fa.STORAGE_F32)
    twin.setup(reuseBuffers=True)
    twin.setInput(x)
    twin.forward()
    twin.finish()
    apart = twin.layers[twin.GEMM].copyResult()
    twin.cleanup()
    assert np.array_equal(got, apart)
