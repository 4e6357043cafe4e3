"""Output stores that are written through the L2 (the 16-position convolution kernels on outputs whose pixels are whole
128-byte lines): such a store does not drop the copies of a line that other XCDs' L2s hold, so the kernels drop them
themselves, once per XCD and launch.  A copy that survived would show as the buffer's previous contents -- the frame
before, the tensor that shared the buffer, the zeros of the allocation -- in a later pass, and only on tensors small
enough to stay in the caches.  The checks: a style net whose tensors fit into one L2 several times over, buffers
shared, a different frame in every pass, every pass bit-identical to the same network with plain stores
(FYNHIP_PLAIN_STORES=1); reference path gpu/deep/deepconvlayerNxN.cpp:129-211 (the result of a layer does not depend
on what its texture held before)."""
import numpy as np
import pytest

import fyusenet_amd as fa
from fyusenet_amd import networks, prng

pytestmark = pytest.mark.gpu


def _passes(net, frames, graph):
    net.setup(reuseBuffers=True)
    infos = {lyr.name: lyr.kernelInfo() for lyr in net.layers}
    outs = []
    net.useGraph(graph)
    for x in frames:
        net.setInput(x)
        net.forward()
        net.finish()
        outs.append(net.getOutput(net.output_layer))
    net.cleanup()
    return outs, infos


@pytest.mark.parametrize("storage", [fa.STORAGE_F32, fa.STORAGE_F16], ids=["f32", "f16"])
@pytest.mark.parametrize("size", [(128, 96), (256, 192)], ids=["128x96", "256x192"])
@pytest.mark.parametrize("graph", [False, True], ids=["eager", "graph"])
def test_written_through_outputs_equal_plain_stores_frame_after_frame(size, graph, storage, monkeypatch):
    w, h = size
    frames = [prng.uniform(4100 + i, (3, h, w), 0.0, 1.0) for i in range(8)]
    frames.insert(4, np.zeros((3, h, w), np.float32))   # (a frame that changes every value)
    monkeypatch.setenv("FYNHIP_FORCE_P16_CONV", "1")
    monkeypatch.delenv("FYNHIP_PLAIN_STORES", raising=False)
    got, infos = _passes(networks.StyleNet(storage, w, h), frames, graph)
    through = [n for n, i in infos.items() if "stores=through" in i]
    print("   written through:", through, flush=True)
    # fp32 tensors: the residual layers, the first two layers and the transposed ones (conv3's two blocks of 64 channels
    # are whole lines as well where its tile choice has them); fp16 tensors: the residual layers run another kernel
    # (conv_h16, plain stores), which leaves the stride-2 layers and, with some tile choices, the first transposed one
    assert len(through) >= (12 if storage == fa.STORAGE_F32 else 2), infos
    monkeypatch.setenv("FYNHIP_PLAIN_STORES", "1")
    want, infos2 = _passes(networks.StyleNet(storage, w, h), frames, graph)
    assert not any("stores=through" in i for i in infos2.values())
    for i, (a, b) in enumerate(zip(got, want)):
        assert np.array_equal(a, b), "pass %d: %d values differ" % (i, int((a != b).sum()))
    assert not np.array_equal(got[0], got[1])


def test_written_through_single_layers_on_a_dirty_buffer(monkeypatch):
    """One 3x3 layer 128 -> 128 at 32x24 run on inputs that alternate between two frames: the output buffer's lines
    are in every L2 that read them for the download of the pass before."""
    monkeypatch.setenv("FYNHIP_FORCE_P16_CONV", "1")
    outs = {}
    for plain in (False, True):
        if plain:
            monkeypatch.setenv("FYNHIP_PLAIN_STORES", "1")
        net = networks.SingleConvNet(fa.STORAGE_F32, channels=128, width=32, height=24)
        net.setup()
        info = net.layers[1].kernelInfo()
        assert ("stores=through" in info) == (not plain), info
        xs = [net.makeInput(), -0.5 * net.makeInput()]
        res = []
        for i in range(10):
            net.setInput(xs[i & 1])
            net.forward()
            net.finish()
            res.append(net.getOutput(net.output_layer))
        net.cleanup()
        outs[plain] = res
    for i in range(10):
        assert np.array_equal(outs[False][i], outs[True][i]), i
    assert not np.array_equal(outs[False][0], outs[False][1])


def test_written_through_outputs_with_several_networks_in_flight(monkeypatch):
    """Four instances of the style net, each with a frame pipeline of its own streams, run side by side (their kernels
    share the XCDs and their L2s, and each launch's workgroups 0..7 drop clean lines under the other instances'
    kernels): every frame equals the plain-store network's synchronous result."""
    monkeypatch.setenv("FYNHIP_FORCE_P16_CONV", "1")
    w, h = 256, 192
    frames = [prng.uniform(6300 + i, (3, h, w), 0.0, 1.0) for i in range(16)]
    monkeypatch.setenv("FYNHIP_PLAIN_STORES", "1")
    want, _ = _passes(networks.StyleNet(fa.STORAGE_F32, w, h), frames, False)
    monkeypatch.delenv("FYNHIP_PLAIN_STORES", raising=False)
    pool = fa.FramePool(lambda: networks.StyleNet(fa.STORAGE_F32, w, h), instances=4, depth=2)
    outs = [np.full_like(want[0], np.nan) for _ in frames]
    tickets = [pool.submit(f, o) for f, o in zip(frames, outs)]
    pool.wait(tickets[-1])
    pool.close()
    for i in range(len(frames)):
        assert np.array_equal(outs[i], want[i]), i
