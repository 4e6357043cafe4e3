"""fyn_layer_copy_result_noalloc (read-back through the library's fixed device array, no allocation) against
fyn_layer_copy_result, bit for bit, through the C ABI: two calls in a row, the second on a smaller tensor, then the
size limit; and that a call leaves the GPU's free memory where it was."""
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


def _allocations(net):
    from fyusenet_amd import capi
    calls, nbytes = ctypes.c_size_t(0), ctypes.c_size_t(0)
    capi.check(capi.lib().fyn_net_device_allocations(net._h, ctypes.byref(calls), ctypes.byref(nbytes)))
    return calls.value, nbytes.value


def _free_device_bytes():
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


@pytest.mark.gpu
def test_no_alloc_read_back_allocates_nothing():
    """What the entry point exists for: on a network whose growable staging area has never been sized, reading back a
    1.6 M-float tensor through it makes no device allocation (the engine's own count of its hipMalloc calls, and the
    GPU's free memory as the runtime reports it), while the allocating entry point, called afterwards on the same
    tensor, makes one of at least the tensor's size."""
    from fyusenet_amd import capi, networks
    net = networks.StyleNet(0, width=256, height=192)   # (the input, 3 channels, sizes the staging area for 147 K floats only)
    net.setup(reuseBuffers=False)
    net.setInput(net.makeInput())
    net.forward()
    net.finish()
    out = np.zeros((32, 192, 256), np.float32)   # the first layer's result: 1.6 M floats
    calls0, bytes0 = _allocations(net)
    free0 = _free_device_bytes()
    for _ in range(2):
        capi.check(capi.lib().fyn_layer_copy_result_noalloc(net._h, 1, capi.fptr(out), 0))
    assert _allocations(net) == (calls0, bytes0)
    assert _free_device_bytes() == free0
    assert out.any()
    want = np.zeros_like(out)
    capi.check(capi.lib().fyn_layer_copy_result(net._h, 1, capi.fptr(want), 0))
    calls1, bytes1 = _allocations(net)
    assert calls1 == calls0 + 1 and bytes1 - bytes0 >= out.nbytes   # (the count sees the staging area being sized)
    assert np.array_equal(out, want)
    net.cleanup()
