"""Python face of the CPU oracle (oracle/fyn_oracle.c) -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py import this module; the
shipped package never does.  It wraps the C restatement with numpy arrays (CHW fp32, unpadded unless
stated) and can execute a whole network description layer by layer.
"""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "_build", "libfynoracle.so")

RESIDUAL_INPUT, RELU_ON_RESIDUAL, BATCHNORM_ON_RESIDUAL, POST_BATCHNORM = 1, 2, 4, 8
PRE_RELU, PRE_CLIP = 64, 128
ACT_NONE, ACT_RELU, ACT_LEAKY, ACT_CLIP = 0, 1, 2, 3

_F = ctypes.POINTER(ctypes.c_float)
_lib = None


def build():
    subprocess.check_call(["make", "-s", "-C", HERE])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = ctypes.CDLL(LIB_PATH)
        for name in ("fyo_conv2d", "fyo_fracconv", "fyo_dwconv", "fyo_transconv", "fyo_gemm", "fyo_maxpool", "fyo_avgpool",
                     "fyo_global_pool", "fyo_batchnorm", "fyo_addsub", "fyo_concat", "fyo_argmax",
                     "fyo_chw_to_deep", "fyo_deep_to_chw", "fyo_shallow_to_chw", "fyo_chw_to_shallow",
                     "fyo_unary", "fyo_scale", "fyo_transpose", "fyo_imgextract", "fyo_nonmax", "fyo_blur",
                     "fyo_blur_coeffs", "fyo_rgb2bgr"):
            getattr(_lib, name).restype = ctypes.c_int
    return _lib


def set_threads(n):
    """Number of OpenMP threads the oracle's loops use (1 = the reference tests' scalar setting)."""
    os.environ["OMP_NUM_THREADS"] = str(n)
    try:
        omp = ctypes.CDLL("libgomp.so.1")
        omp.omp_set_num_threads(int(n))
    except OSError:
        pass


def _f(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_F)


def _act(act):
    """act = (kind, leak, lo, hi) or None."""
    if act is None:
        return (ACT_NONE, 0.0, 0.0, 0.0)
    return act


def pad_chw(x, pad):
    return np.pad(x, ((0, 0), (pad, pad), (pad, pad))) if pad else x


def conv2d(x_stored, pad_in, block, cout, k, dil=1, stride=1, act=None, flags=0, residual=None, border=0):
    """x_stored [cin][H+2pad][W+2pad]; returns [cout][H/stride][W/stride]."""
    x, xp = _f(x_stored)
    b, bp = _f(block)
    cin, hs, ws = x.shape
    ho, wo = (hs - 2 * pad_in) // stride, (ws - 2 * pad_in) // stride
    out = np.empty((cout, ho, wo), dtype=np.float32)
    r, rp = (None, None) if residual is None else _f(residual)
    a = _act(act)
    rc = lib().fyo_conv2d(xp, cin, hs, ws, pad_in, bp, cout, k, dil, stride, a[0], ctypes.c_float(a[1]),
                          ctypes.c_float(a[2]), ctypes.c_float(a[3]), ctypes.c_uint(flags), rp, border,
                          out.ctypes.data_as(_F))
    assert rc == 0
    return out


def fracconv(x_stored, pad_in, block, cout, k, stride=1, inv_step=2, act=None, flags=0, residual=None, border=1):
    """x_stored [cin][H+2pad][W+2pad]; returns [cout][H*inv_step/stride][W*inv_step/stride]."""
    x, xp = _f(x_stored)
    b, bp = _f(block)
    cin, hs, ws = x.shape
    ho, wo = (hs - 2 * pad_in) * inv_step // stride, (ws - 2 * pad_in) * inv_step // stride
    out = np.empty((cout, ho, wo), dtype=np.float32)
    r, rp = (None, None) if residual is None else _f(residual)
    a = _act(act)
    rc = lib().fyo_fracconv(xp, cin, hs, ws, pad_in, bp, cout, k, stride, inv_step, a[0], ctypes.c_float(a[1]),
                            ctypes.c_float(a[2]), ctypes.c_float(a[3]), ctypes.c_uint(flags), rp, border,
                            out.ctypes.data_as(_F))
    assert rc == 0, rc
    return out


def dwconv(x_stored, pad_in, block, mult=1, k=3, dil=1, stride=1, act=None, flags=0, residual=None):
    x, xp = _f(x_stored)
    b, bp = _f(block)
    cin, hs, ws = x.shape
    ho, wo = (hs - 2 * pad_in) // stride, (ws - 2 * pad_in) // stride
    out = np.empty((cin * mult, ho, wo), dtype=np.float32)
    r, rp = (None, None) if residual is None else _f(residual)
    a = _act(act)
    rc = lib().fyo_dwconv(xp, cin, hs, ws, pad_in, bp, mult, k, dil, stride, a[0], ctypes.c_float(a[1]),
                          ctypes.c_float(a[2]), ctypes.c_float(a[3]), ctypes.c_uint(flags), rp, out.ctypes.data_as(_F))
    assert rc == 0
    return out


def transconv(x_stored, pad_in, block, cout, k, crop=0, act=None, flags=0, residual=None):
    x, xp = _f(x_stored)
    b, bp = _f(block)
    cin, hs, ws = x.shape
    h, w = hs - 2 * pad_in, ws - 2 * pad_in
    out = np.empty((cout, 2 * h + k - 2 - crop, 2 * w + k - 2 - crop), dtype=np.float32)
    r, rp = (None, None) if residual is None else _f(residual)
    a = _act(act)
    rc = lib().fyo_transconv(xp, cin, hs, ws, pad_in, bp, cout, k, crop, a[0], ctypes.c_float(a[1]),
                             ctypes.c_float(a[2]), ctypes.c_float(a[3]), ctypes.c_uint(flags), rp,
                             out.ctypes.data_as(_F))
    assert rc == 0
    return out


def gemm(x, block, cout, act=None, flags=0):
    xv, xp = _f(np.asarray(x).reshape(-1))
    b, bp = _f(block)
    out = np.empty((cout,), dtype=np.float32)
    a = _act(act)
    rc = lib().fyo_gemm(xp, xv.size, bp, cout, a[0], ctypes.c_float(a[1]), ctypes.c_float(a[2]), ctypes.c_float(a[3]),
                        ctypes.c_uint(flags), out.ctypes.data_as(_F))
    assert rc == 0
    return out


def _pool(fn, x_stored, pad_in, pool, stride, act):
    x, xp = _f(x_stored)
    c, hs, ws = x.shape
    ho, wo = (hs - 2 * pad_in) // stride, (ws - 2 * pad_in) // stride
    out = np.empty((c, ho, wo), dtype=np.float32)
    a = _act(act)
    rc = fn(xp, c, hs, ws, pad_in, pool, stride, a[0], ctypes.c_float(a[1]), ctypes.c_float(a[2]), ctypes.c_float(a[3]),
            out.ctypes.data_as(_F))
    assert rc == 0
    return out


def maxpool(x_stored, pad_in, pool, stride, act=None):
    return _pool(lib().fyo_maxpool, x_stored, pad_in, pool, stride, act)


def avgpool(x_stored, pad_in, pool, stride, act=None):
    return _pool(lib().fyo_avgpool, x_stored, pad_in, pool, stride, act)


def global_pool(x_stored, pad_in, is_max, act=None):
    x, xp = _f(x_stored)
    c, hs, ws = x.shape
    out = np.empty((c,), dtype=np.float32)
    a = _act(act)
    rc = lib().fyo_global_pool(xp, c, hs, ws, pad_in, 1 if is_max else 0, a[0], ctypes.c_float(a[1]),
                               ctypes.c_float(a[2]), ctypes.c_float(a[3]), out.ctypes.data_as(_F))
    assert rc == 0
    return out.reshape(c, 1, 1)


def batchnorm(x_stored, pad_in, sb, act=None, flags=0, residual=None):
    x, xp = _f(x_stored)
    s, sp = _f(sb)
    c, hs, ws = x.shape
    out = np.empty((c, hs - 2 * pad_in, ws - 2 * pad_in), dtype=np.float32)
    r, rp = (None, None) if residual is None else _f(residual)
    a = _act(act)
    rc = lib().fyo_batchnorm(xp, c, hs, ws, pad_in, sp, a[0], ctypes.c_float(a[1]), ctypes.c_float(a[2]),
                             ctypes.c_float(a[3]), ctypes.c_uint(flags), rp, out.ctypes.data_as(_F))
    assert rc == 0
    return out


def addsub(a_, b_, sub=False, act=None):
    a1, ap = _f(a_)
    b1, bp = _f(b_)
    out = np.empty_like(a1)
    a = _act(act)
    lib().fyo_addsub(ap, bp, ctypes.c_size_t(a1.size), 1 if sub else 0, a[0], ctypes.c_float(a[1]), ctypes.c_float(a[2]),
                     ctypes.c_float(a[3]), out.ctypes.data_as(_F))
    return out


def concat(inputs, act=None):
    arrs = [np.ascontiguousarray(i, dtype=np.float32) for i in inputs]
    h, w = arrs[0].shape[1:]
    ptrs = (_F * len(arrs))(*[a.ctypes.data_as(_F) for a in arrs])
    chans = (ctypes.c_int * len(arrs))(*[a.shape[0] for a in arrs])
    out = np.empty((sum(a.shape[0] for a in arrs), h, w), dtype=np.float32)
    a = _act(act)
    lib().fyo_concat(ptrs, chans, len(arrs), h, w, a[0], ctypes.c_float(a[1]), ctypes.c_float(a[2]), ctypes.c_float(a[3]),
                     out.ctypes.data_as(_F))
    return out


def argmax(x, act=None):
    xv, xp = _f(x)
    c, h, w = xv.shape
    idx = np.empty((h, w), dtype=np.int32)
    val = np.empty((h, w), dtype=np.float32)
    a = _act(act)
    lib().fyo_argmax(xp, c, h, w, a[0], ctypes.c_float(a[1]), ctypes.c_float(a[2]), ctypes.c_float(a[3]),
                     idx.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), val.ctypes.data_as(_F))
    return idx, val


FN_COPY, FN_SIGMOID, FN_TANH, FN_ARITH, FN_CAST = 0, 1, 2, 3, 4


def unary(x, fn, op=0, operand=0.0, act=None):
    """Element-wise function layer on an unpadded tensor: copy / sigmoid / tanh / singleton arithmetic / cast."""
    xv, xp = _f(x)
    out = np.empty_like(xv)
    a = _act(act)
    rc = lib().fyo_unary(xp, ctypes.c_size_t(xv.size), fn, op, ctypes.c_float(operand), a[0], ctypes.c_float(a[1]),
                         ctypes.c_float(a[2]), ctypes.c_float(a[3]), out.ctypes.data_as(_F))
    assert rc == 0
    return out


def scale(x_stored, pad_in, up=(1, 1), down=(1, 1), linear=False, deep=True, act=None):
    """Scale layer; up/down = (x, y) integer factors.  x_stored [c][H+2pad][W+2pad]."""
    x, xp = _f(x_stored)
    c, hs, ws = x.shape
    h, w = hs - 2 * pad_in, ws - 2 * pad_in
    out = np.empty((c, h * up[1] // down[1], w * up[0] // down[0]), dtype=np.float32)
    a = _act(act)
    rc = lib().fyo_scale(xp, c, hs, ws, pad_in, up[0], up[1], down[0], down[1], 1 if linear else 0, 1 if deep else 0,
                         a[0], ctypes.c_float(a[1]), ctypes.c_float(a[2]), ctypes.c_float(a[3]), out.ctypes.data_as(_F))
    assert rc == 0
    return out


def transpose(x, act=None):
    xv, xp = _f(x)
    c, h, w = xv.shape
    out = np.empty((c, w, h), dtype=np.float32)
    a = _act(act)
    rc = lib().fyo_transpose(xp, c, h, w, a[0], ctypes.c_float(a[1]), ctypes.c_float(a[2]), ctypes.c_float(a[3]),
                             out.ctypes.data_as(_F))
    assert rc == 0
    return out


def imgextract(x, window, cout, act=None):
    xv, xp = _f(x)
    c, h, w = xv.shape
    out = np.empty((cout, h // window, w // window), dtype=np.float32)
    a = _act(act)
    rc = lib().fyo_imgextract(xp, c, h, w, window, cout, a[0], ctypes.c_float(a[1]), ctypes.c_float(a[2]),
                              ctypes.c_float(a[3]), out.ctypes.data_as(_F))
    assert rc == 0
    return out


def nonmax(x_stored, pad_in):
    x, xp = _f(x_stored)
    c, hs, ws = x.shape
    out = np.empty((c, hs - 2 * pad_in, ws - 2 * pad_in), dtype=np.float32)
    assert lib().fyo_nonmax(xp, c, hs, ws, pad_in, out.ctypes.data_as(_F)) == 0
    return out


def blur_coeffs(k, gaussian):
    out = np.empty((k, k), dtype=np.float32)
    assert lib().fyo_blur_coeffs(k, 1 if gaussian else 0, out.ctypes.data_as(_F)) == 0
    return out


def blur(x_stored, pad_in, k, gaussian=False):
    x, xp = _f(x_stored)
    c, hs, ws = x.shape
    out = np.empty((c, hs - 2 * pad_in, ws - 2 * pad_in), dtype=np.float32)
    assert lib().fyo_blur(xp, c, hs, ws, pad_in, k, 1 if gaussian else 0, out.ctypes.data_as(_F)) == 0
    return out


def rgb2bgr(x):
    xv, xp = _f(x)
    c, h, w = xv.shape
    out = np.empty_like(xv)
    assert lib().fyo_rgb2bgr(xp, c, h, w, out.ctypes.data_as(_F)) == 0
    return out


def round_fp16(x):
    xv, xp = _f(x)
    out = np.empty_like(xv)
    lib().fyo_round_fp16.restype = None
    lib().fyo_round_fp16(xp, ctypes.c_size_t(xv.size), out.ctypes.data_as(_F))
    return out


def deep_tiling(channels):
    tx, ty = ctypes.c_int(), ctypes.c_int()
    lib().fyo_deep_tiling.restype = None
    lib().fyo_deep_tiling(channels, ctypes.byref(tx), ctypes.byref(ty))
    return tx.value, ty.value


def chw_to_deep(x, pad):
    xv, xp = _f(x)
    c, h, w = xv.shape
    tx, ty = deep_tiling(c)
    out = np.empty((ty * (h + pad) + pad, tx * (w + pad) + pad, 4), dtype=np.float32)
    lib().fyo_chw_to_deep(xp, c, h, w, pad, out.ctypes.data_as(_F))
    return out


def deep_to_chw(deep, c, h, w, pad):
    dv, dp = _f(deep)
    out = np.empty((c, h, w), dtype=np.float32)
    lib().fyo_deep_to_chw(dp, c, h, w, pad, out.ctypes.data_as(_F))
    return out


def chw_to_shallow(x, pc):
    xv, xp = _f(x)
    c, h, w = xv.shape
    out = np.empty((h, w, pc), dtype=np.float32)
    lib().fyo_chw_to_shallow(xp, c, h, w, pc, out.ctypes.data_as(_F))
    return out


def shallow_to_chw(hwc, c):
    hv, hp = _f(hwc)
    h, w, pc = hv.shape
    out = np.empty((c, h, w), dtype=np.float32)
    lib().fyo_shallow_to_chw(hp, c, h, w, pc, out.ctypes.data_as(_F))
    return out


# ---------------------------------------------------------------------------------------------
# whole-network execution from a description (NeuralNetwork.describe() of the package)
# ---------------------------------------------------------------------------------------------
def _builder_act(b, flags):
    if flags & PRE_RELU:
        leak = float(getattr(b, "leakyReLU_", 0.0)) if int(b.preAct_) == 2 else 0.0
        return (ACT_LEAKY, leak, 0.0, 0.0) if leak != 0.0 else (ACT_RELU, 0.0, 0.0, 0.0)
    if flags & PRE_CLIP:
        return (ACT_CLIP, 0.0, float(b.clipLow_), float(b.clipHigh_))
    return None


def _round_block_fp16(layer_type, b, block):
    """fp16 storage rounds the weights (not bias / BN terms, which the engine keeps in fp32)."""
    block = np.array(block, dtype=np.float32, copy=True)
    cout = b.outputChannels_
    if layer_type in (6, 7, 8, 31):  # conv, fractional conv, transconv, gemm
        dw = layer_type == 6 and getattr(b, "groupSize_", 1) not in (0, 1) and b.groupSize_ == b.inputChannels_
        if dw:
            return block  # depthwise weights stay fp32 in the engine
        k = getattr(b, "kernel_", 1) if layer_type != 31 else 1
        n = cout * k * k * b.inputChannels_
        block[cout:cout + n] = round_fp16(block[cout:cout + n])
    return block


def run_layer(b, w, ins, f16=False):
    """One layer on the CPU.  b: builder, w: weight block, ins: unpadded CHW input per port.
    Returns the unpadded CHW output (not yet rounded to the storage type)."""
    t = int(b.type_)
    flags = int(b.getFlags())
    act = _builder_act(b, flags)

    def get(port, pad):
        return pad_chw(np.asarray(ins[port], dtype=np.float32), pad)

    if t in (26, 27):  # download / upload: pass-through
        return np.asarray(ins[0], dtype=np.float32)
    if t == 6:
        res = get(1, 0) if flags & RESIDUAL_INPUT else None
        wb = _round_block_fp16(t, b, w) if f16 else w
        dw = getattr(b, "groupSize_", 1) not in (0, 1) and b.groupSize_ == b.inputChannels_
        if dw:
            return dwconv(get(0, b.inputPadding_), b.inputPadding_, wb, 1, b.kernel_, b.dilation_[0], b.downsample_[0], act, flags, res)
        r = (b.kernel_ - 1) // 2 * b.dilation_[0]
        border = 1 if (not (flags & 16) and b.inputPadding_ < r and b.kernel_ > 1) else 0
        return conv2d(get(0, b.inputPadding_), b.inputPadding_, wb, b.outputChannels_, b.kernel_, b.dilation_[0],
                      b.downsample_[0], act, flags, res, border)
    if t == 7:
        res = get(1, 0) if flags & RESIDUAL_INPUT else None
        wb = _round_block_fp16(t, b, w) if f16 else w
        inv = int(round(1.0 / b.sourceStep_))
        return fracconv(get(0, b.inputPadding_), b.inputPadding_, wb, b.outputChannels_, b.kernel_, b.downsample_[0], inv, act, flags, res)
    if t == 8:
        wb = _round_block_fp16(t, b, w) if f16 else w
        return transconv(get(0, b.inputPadding_), b.inputPadding_, wb, b.outputChannels_, b.kernel_, b.transconvCrop_, act, flags)
    if t == 31:
        wb = _round_block_fp16(t, b, w) if f16 else w
        return gemm(get(0, 0), wb, b.outputChannels_, act, flags).reshape(-1, 1, 1)
    if t in (9, 10):
        if b.global_:
            return global_pool(get(0, b.inputPadding_), b.inputPadding_, t == 10, act)
        if t == 10:
            return maxpool(get(0, b.inputPadding_), b.inputPadding_, b.poolsize_[0], b.downsample_[0], act)
        return avgpool(get(0, b.inputPadding_), b.inputPadding_, b.poolsize_[0], b.downsample_[0], act)
    if t == 30:
        res = get(1, 0) if flags & RESIDUAL_INPUT else None
        return batchnorm(get(0, 0), 0, w, act, flags, res)
    if t in (1, 2):
        return addsub(get(0, 0), get(1, 0), t == 2, act)
    if t == 5:
        all_relu = all(f & PRE_RELU for (_, _, f) in b.inputs_)
        a = act if act is not None else ((ACT_RELU, 0.0, 0.0, 0.0) if all_relu else None)
        return concat([get(p, 0) for p in range(len(b.inputs_))], a)
    if t == 3:
        idx, val = argmax(get(0, 0), act)
        return np.stack([idx.astype(np.float32), val])
    if t in (11, 12, 14, 15, 24, 25):   # padding / scale / relu / clip / deep<->shallow: all a scale layer
        deep = bool(flags & 16)
        linear = int(getattr(b, "scaleType_", 0)) == 1
        if deep and (b.width_ == 1 or b.height_ == 1):
            linear = False                  # gpu/deep/deepscalelayer.cpp:44
        return scale(get(0, b.inputPadding_), b.inputPadding_, tuple(b.upsample_), tuple(b.downsample_), linear, deep, act)
    if t == 17:
        return unary(get(0, 0), FN_SIGMOID, act=act)
    if t == 16:
        return unary(get(0, 0), FN_TANH, act=act)
    if t == 13:
        return unary(get(0, 0), FN_ARITH, int(b.opType_), float(b.operand_), act)
    if t == 4:
        return unary(get(0, 0), FN_CAST, int(b.target_), act=act)
    if t == 19:
        return transpose(get(0, 0), act)
    if t == 20:
        return imgextract(get(0, 0), b.window_, b.outputChannels_, act)
    if t == 22:
        return nonmax(get(0, b.inputPadding_), b.inputPadding_)
    if t == 21:
        return blur(get(0, b.inputPadding_), b.inputPadding_, b.kernel_, int(b.blurType_) == 1)
    if t == 23:
        return rgb2bgr(get(0, 0))
    raise ValueError("oracle: unsupported layer type %d" % t)


def num_ports(b):
    t = int(b.type_)
    if t == 27:
        return 1  # fed from the host
    if t == 5:
        return len(b.inputs_)
    if t in (1, 2):
        return 2
    return 2 if int(b.getFlags()) & RESIDUAL_INPUT else 1


def port_channels(b, port):
    """Channels a layer expects on an input port, None when the builder does not say."""
    if int(b.type_) == 5:                                  # concatenation: per-input channel counts
        ins = getattr(b, "inputs_", None)
        return ins[port][0] if ins and port < len(ins) else None
    if port == 0:
        return b.inputChannels_
    return b.outputChannels_ if port == 1 else None       # residual input


def run_network(desc, inputs, fp16_storage=None, forced=None, known=None, only=None):
    """Executes a network description on the CPU.

    desc: NeuralNetwork.describe(); inputs: {(layer_number, port): CHW array} for upload layers
    (port 0) and unconnected ports.  Returns {layer_number: CHW output (unpadded)}.
    fp16_storage: emulate fp16 tensors/weights (default: desc['storage'] == 1).
    forced: optional {layer_number: CHW array}; when given, every layer reads these tensors instead of
    the oracle's own upstream results (per-layer check on identical inputs).
    known / only: evaluate a part of the graph: `only` is the set of layer numbers to run, `known` holds the tensors
    that this part reads from layers outside it ({layer_number: CHW array}).
    """
    f16 = (desc.get("storage", 0) == 1) if fp16_storage is None else fp16_storage
    rnd = round_fp16 if f16 else (lambda a: np.asarray(a, dtype=np.float32))
    feeds = {}
    for (src, dst, port) in desc["connections"]:
        feeds[(dst, port)] = src
    outs = dict(known) if known else {}
    for entry in sorted(desc["layers"], key=lambda e: e["number"]):
        b, no, w = entry["builder"], entry["number"], entry["weights"]
        if only is not None and no not in only:
            continue
        ins = []
        for port in range(num_ports(b)):
            if (no, port) in feeds:
                src = feeds[(no, port)]
                x = forced[src] if forced is not None else outs[src]
                want = port_channels(b, port)
                if want is not None and want != x.shape[0] and (want + 3) // 4 == (x.shape[0] + 3) // 4:
                    # the consumer names another channel count inside the same group of four (buffers are matched
                    # texture by texture, base/buffermanager.cpp:476): missing channels read as zero
                    x = np.concatenate([x, np.zeros((want - x.shape[0],) + x.shape[1:], x.dtype)]) if want > x.shape[0] else x[:want]
                ins.append(x)
            else:
                ins.append(rnd(inputs[(no, port)]))
        outs[no] = rnd(run_layer(b, w, ins, f16))
    return outs
