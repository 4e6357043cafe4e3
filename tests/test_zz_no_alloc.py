"""fyn_layer_copy_result_noalloc (read-back through the library's fixed device array, no allocation) against
fyn_layer_copy_result, bit for bit, through the C ABI: two calls in a row, the second on a smaller tensor, then the
size limit."""
import ctypes

import numpy as np
import pytest

STATIC_SCRATCH_FLOATS = 8 << 20   # FYN_STATIC_SCRATCH_FLOATS of include/fynhip.h


def _both(net, layer_no, include_padding):
    from fyusenet_amd import capi
    c, h, w, p = net.layers[layer_no].outputShape()
    if include_padding:
        h, w = h + 2 * p, w + 2 * p
    want = np.full((c, h, w), np.nan, np.float32)
    got = np.full((c, h, w), np.nan, np.float32)
    capi.check(capi.lib().fyn_layer_copy_result(net._h, layer_no, capi.fptr(want), int(include_padding)))
    capi.check(capi.lib().fyn_layer_copy_result_noalloc(net._h, layer_no, capi.fptr(got), int(include_padding)))
    return got, want


@pytest.mark.gpu
@pytest.mark.parametrize("storage", [0, 1])
def test_no_alloc_read_back_equals_copy_result(storage):
    from fyusenet_amd import capi, networks
    net = networks.StyleNet(storage, width=96, height=64)
    net.setup(reuseBuffers=False)   # every layer's tensor stays readable
    net.setInput(net.makeInput())
    net.forward()
    net.finish()
    print("case: style net 96x64 storage=%d" % storage, flush=True)
    # first call: the largest tensor (32 channels at full size, with its halo); second: a smaller one; third: larger again
    order = [(1, True), (3, False), (net.last_conv, False), (2, True)]
    sizes = []
    for layer_no, pad in order:
        got, want = _both(net, layer_no, pad)
        assert np.isfinite(want).all() and want.std() > 0
        assert np.array_equal(got, want), (layer_no, pad)
        sizes.append(got.size)
    assert sizes[1] < sizes[0] and sizes[2] < sizes[1] and sizes[3] > sizes[2]
    net.cleanup()


@pytest.mark.gpu
def test_no_alloc_read_back_refuses_what_does_not_fit():
    from fyusenet_amd import capi, networks
    side = 384   # 64 x 384 x 384 = 9.4 M floats > 8 Mi
    net = networks.SingleConvNet(0, size=side)
    net.setup()
    net.setInput(net.makeInput())
    net.forward()
    net.finish()
    assert 64 * side * side > STATIC_SCRATCH_FLOATS
    out = np.zeros((64, side, side), np.float32)
    rc = capi.lib().fyn_layer_copy_result_noalloc(net._h, 1, capi.fptr(out), 0)
    assert rc == -1   # FYN_ERR_INVALID
    msg = capi.lib().fyn_last_error().decode()
    assert "fixed staging area" in msg and "fyn_layer_copy_result" in msg
    assert not out.any()
    # the allocating entry point still serves it
    capi.check(capi.lib().fyn_layer_copy_result(net._h, 1, capi.fptr(out), 0))
    assert out.any()
    net.cleanup()
