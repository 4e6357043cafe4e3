"""NeuralNetwork / LayerFactory / BufferManager surface on top of the C ABI.

Mirrors the way the reference's networks are written (samples/samplenetworks/resnet50.cpp:200-536):
a NeuralNetwork subclass implements buildLayers() (builders pushed into a LayerFactory),
connectLayers(layers, bufferManager) and initializeWeights(layers); setup() runs them in the order
of NeuralNetwork::glSetup (fyusenet/base/neuralnetwork.cpp:238-250).
"""
import ctypes
import os

import numpy as np

from . import capi
from .builders import LayerType


class Layer:
    """Handle of one compiled layer (LayerBase / GPULayerBase of the reference)."""

    def __init__(self, net, builder):
        self._net = net
        self.builder = builder
        self.number = builder.number_
        self.name = builder.name_
        self.weights = None  # host copy of the loaded block (kept for descriptions handed to checkers)

    def getNumber(self):
        return self.number

    def getName(self):
        return self.name

    def loadWeightsAndBiases(self, data, offset=0):
        """ConvLayerInterface::loadWeightsAndBiases (base/convlayerinterface.h:95)."""
        data = np.ascontiguousarray(data, dtype=np.float32)
        n = self.weightFloats()
        if offset + n > data.size:
            raise capi.FynException(capi.ERR_INVALID, "weight block of layer %s exceeds the supplied array" % self.name)
        self.weights = data[offset:offset + n].copy()
        capi.check(capi.lib().fyn_layer_load_weights(self._net._h, self.number, capi.fptr(data), offset))

    def loadScaleAndBias(self, data, offset=0):
        """BatchNormInterface::loadScaleAndBias (base/batchnorminterface.h:146)."""
        data = np.ascontiguousarray(data, dtype=np.float32)
        n = self.weightFloats()
        if offset + n > data.size:
            raise capi.FynException(capi.ERR_INVALID, "scale/bias block of layer %s exceeds the supplied array" % self.name)
        self.weights = data[offset:offset + n].copy()
        capi.check(capi.lib().fyn_layer_load_scale_bias(self._net._h, self.number, capi.fptr(data), offset))

    def weightFloats(self):
        n = ctypes.c_size_t(0)
        capi.check(capi.lib().fyn_layer_weight_floats(self._net._h, self.number, ctypes.byref(n)))
        return n.value

    def outputShape(self):
        c, h, w, p = ctypes.c_int(), ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
        capi.check(capi.lib().fyn_layer_output_shape(self._net._h, self.number, ctypes.byref(c), ctypes.byref(h),
                                                     ctypes.byref(w), ctypes.byref(p)))
        return c.value, h.value, w.value, p.value

    def copyResult(self, includePadding=False):
        """GPULayerBase::copyResult (gpu/gpulayerbase.cpp:525-564): CHW fp32."""
        c, h, w, p = self.outputShape()
        if includePadding:
            h, w = h + 2 * p, w + 2 * p
        out = np.empty((c, h, w), dtype=np.float32)
        capi.check(capi.lib().fyn_layer_copy_result(self._net._h, self.number, capi.fptr(out), 1 if includePadding else 0))
        return out

    def setInput(self, data, port=0, order=capi.ORDER_CHANNELWISE):
        data = np.ascontiguousarray(data, dtype=np.float32)
        want = ctypes.c_size_t(0)
        capi.check(capi.lib().fyn_net_input_floats(self._net._h, self.number, port, ctypes.byref(want)))
        if data.size != want.value:
            raise capi.FynException(capi.ERR_INVALID, "input of layer %s, port %d, takes %d floats, the buffer holds %d" % (self.name, port, want.value, data.size))
        capi.check(capi.lib().fyn_net_set_input(self._net._h, self.number, port, capi.fptr(data), order))

    def kernelInfo(self):
        buf = ctypes.create_string_buffer(512)
        capi.check(capi.lib().fyn_layer_kernel_info(self._net._h, self.number, buf, len(buf)))
        return buf.value.decode()

    def timeKernel(self, iters):
        ms = ctypes.c_float(0)
        capi.check(capi.lib().fyn_layer_time(self._net._h, self.number, iters, ctypes.byref(ms)))
        return ms.value / iters


class CompiledLayers:
    """base/compiledlayers.h:50-291: number- and name-indexed layer store, ascending iteration."""

    def __init__(self):
        self._by_number = {}
        self._by_name = {}

    def _add(self, layer):
        self._by_number[layer.number] = layer
        self._by_name[layer.name] = layer

    def __getitem__(self, key):
        try:
            return self._by_name[key] if isinstance(key, str) else self._by_number[key]
        except KeyError:
            raise capi.FynException(capi.ERR_NOTFOUND, "no layer %r" % (key,))

    def __iter__(self):
        return iter(self._by_number[k] for k in sorted(self._by_number))

    def __len__(self):
        return len(self._by_number)


class LayerFactory:
    """base/layerfactory.h:56-138."""

    def __init__(self, net):
        self._net = net
        self._builders = {}

    def pushBuilder(self, builder):
        # base/layerfactory.cpp:67-76
        if builder.number_ < 0:
            raise capi.FynException(capi.ERR_INVALID, "Must identify each layer with a valid number (found %d in the builder)" % builder.number_)
        if int(builder.type_) >= int(LayerType.LAST_SUPPORTED):
            raise capi.FynException(capi.ERR_UNSUPPORTED, "Unsupported layer type %d" % int(builder.type_))
        if builder.number_ in self._builders:
            raise capi.FynException(capi.ERR_DUPLICATE, "Trying to insert a layer on a position that is already taken (%d)" % builder.number_)
        self._builders[builder.number_] = builder

    def _add_custom(self, b, d):
        # gpu/gpulayerfactory.cpp:586-589: the builder's callback creates the layer
        if not hasattr(b, "init"):
            raise capi.FynException(capi.ERR_INVALID, "layer %s: a CUSTOM layer needs a CustomLayerBuilder with its init callback" % b.name_)
        impl = b.init()
        thunks = _custom_thunks(impl)
        self._net._keepalive.append((impl, thunks))     # the engine calls them until the network is destroyed
        c = capi.CustomLayer(None, *thunks)
        capi.check(capi.lib().fyn_net_add_custom_layer(self._net._h, ctypes.byref(d), ctypes.byref(c)))

    def compileLayers(self):
        layers = CompiledLayers()
        for no in sorted(self._builders):
            b = self._builders[no]
            d = b.desc()
            if int(b.type_) == int(LayerType.CUSTOM):
                self._add_custom(b, d)
            else:
                capi.check(capi.lib().fyn_net_add_layer(self._net._h, ctypes.byref(d)))
            layers._add(Layer(self._net, b))
        return layers


def _custom_thunks(impl):
    """C callbacks around a Python custom-layer object; exceptions become a non-zero status."""
    def views(ptr, n):
        return [ptr[i] for i in range(n)]

    def setup(_user, ins, n, out):
        try:
            if hasattr(impl, "setup"):
                impl.setup(views(ins, n), out[0])
            return 0
        except Exception:   # noqa: BLE001 -- must not propagate through the C frame
            return 1

    def forward(_user, ins, n, out, stream, seq):
        try:
            impl.forward(views(ins, n), out[0], stream or 0, seq)
            return 0
        except Exception:   # noqa: BLE001
            return 1

    def cleanup(_user):
        try:
            if hasattr(impl, "cleanup"):
                impl.cleanup()
        except Exception:   # noqa: BLE001
            pass

    return capi.CUSTOM_SETUP_FN(setup), capi.CUSTOM_FORWARD_FN(forward), capi.CUSTOM_CLEANUP_FN(cleanup)


class BufferManager:
    """base/buffermanager.cpp:160-184 (connectLayers); tensors live in the engine."""

    def __init__(self, net):
        self._net = net
        self.connections = []

    def connectLayers(self, outputLayer, inputLayer, port=0):
        capi.check(capi.lib().fyn_net_connect(self._net._h, outputLayer.number, inputLayer.number, port))
        self.connections.append((outputLayer.number, inputLayer.number, port))


class NeuralNetwork:
    """base/neuralnetwork.h:62-261.  storage: capi.STORAGE_F32 (HIGH_PRECISION) or STORAGE_F16."""

    def __init__(self, storage=capi.STORAGE_F32, device=0):
        self.storage = storage
        self._keepalive = []   # custom-layer objects and their C thunks
        self._h = ctypes.c_void_p()
        capi.check(capi.lib().fyn_net_create(device, storage, ctypes.byref(self._h)))
        self.layers = None
        self.bufferManager = None
        self._setup = False

    # -- to be provided by the network description --
    def buildLayers(self, factory):
        raise NotImplementedError

    def connectLayers(self, layers, bufferManager):
        raise NotImplementedError

    def initializeWeights(self, layers):
        pass

    # -- life cycle --
    def setup(self, reuseBuffers=True):
        if self._setup:
            raise capi.FynException(capi.ERR_STATE, "network is already set up")
        capi.check(capi.lib().fyn_net_set_buffer_reuse(self._h, 1 if reuseBuffers else 0))
        factory = LayerFactory(self)
        self.buildLayers(factory)
        self.layers = factory.compileLayers()
        self.bufferManager = BufferManager(self)
        self.connectLayers(self.layers, self.bufferManager)
        self.initializeWeights(self.layers)
        capi.check(capi.lib().fyn_net_setup(self._h))
        self._setup = True

    def forward(self):
        seq = ctypes.c_uint64(0)
        capi.check(capi.lib().fyn_net_forward(self._h, ctypes.byref(seq)))
        return seq.value

    def finish(self):
        capi.check(capi.lib().fyn_net_finish(self._h))

    def cleanup(self):
        if self._h:
            capi.check(capi.lib().fyn_net_destroy(self._h))
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.cleanup()
        except Exception:
            pass

    # -- I/O and instrumentation --
    def getOutput(self, layer, order=capi.ORDER_CHANNELWISE):
        lyr = self.layers[layer] if not isinstance(layer, Layer) else layer
        c, h, w, p = lyr.outputShape()
        if order == capi.ORDER_CHANNELWISE:
            out = np.empty((c, h, w), dtype=np.float32)
        elif order == capi.ORDER_GPU_SHALLOW:
            out = np.empty((h, w, 4 if c == 3 else c), dtype=np.float32)
        else:
            from .formats import deep_tiling
            tx, ty = deep_tiling(c)
            out = np.empty((ty * (h + p) + p, tx * (w + p) + p, 4), dtype=np.float32)
        capi.check(capi.lib().fyn_net_get_output(self._h, lyr.number, capi.fptr(out), order))
        return out

    def getArgMax(self, layer):
        lyr = self.layers[layer] if not isinstance(layer, Layer) else layer
        c, h, w, p = lyr.outputShape()
        idx = np.empty((h, w), dtype=np.int32)
        val = np.empty((h, w), dtype=np.float32)
        capi.check(capi.lib().fyn_layer_copy_argmax(self._h, lyr.number, idx.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)), capi.fptr(val)))
        return idx, val

    def enableTimings(self, enable=True):
        capi.check(capi.lib().fyn_net_enable_timings(self._h, 1 if enable else 0))

    def getTiming(self, layer):
        ms, runs = ctypes.c_float(0), ctypes.c_int(0)
        capi.check(capi.lib().fyn_net_get_timing(self._h, layer, ctypes.byref(ms), ctypes.byref(runs)))
        return ms.value, runs.value

    def enableIntermediateOutput(self, directory):
        capi.check(capi.lib().fyn_net_enable_intermediate_output(self._h, directory.encode() if directory else None))

    def useGraph(self, enable=True):
        capi.check(capi.lib().fyn_net_use_graph(self._h, 1 if enable else 0))

    def timeSteps(self, iters):
        """GPU time of each of `iters` forward passes queued back to back (events on the network's stream), ms."""
        ms = np.zeros(iters, np.float32)
        capi.check(capi.lib().fyn_net_time_steps(self._h, iters, capi.fptr(ms)))
        return ms

    def timeForward(self, iters):
        ms = ctypes.c_float(0)
        capi.check(capi.lib().fyn_net_time_forward(self._h, iters, ctypes.byref(ms)))
        return ms.value

    # -- frame pipeline (asynchronous engine mode of the reference, base/engine.cpp:386-683) --
    def asyncBegin(self, inLayer, outLayer, inOrder=capi.ORDER_CHANNELWISE, outOrder=capi.ORDER_CHANNELWISE, depth=2, inPort=0, copyStreams=True):
        """copyStreams=False queues uploads and downloads on the network's own stream (for networks that run side by
        side, see FramePool)."""
        capi.check(capi.lib().fyn_net_async_begin(self._h, inLayer, inPort, inOrder, outLayer, outOrder, depth, 1 if copyStreams else 0))
        a, b = ctypes.c_size_t(0), ctypes.c_size_t(0)
        capi.check(capi.lib().fyn_net_async_sizes(self._h, ctypes.byref(a), ctypes.byref(b)))
        self._async_sizes = (a.value, b.value)
        self._async_outs = {}   # ticket -> output array, kept alive until the engine has written it

    def asyncSubmit(self, frame, out):
        """Queues one frame; `out` (a C-contiguous float32 array) is filled once asyncWait(ticket) has returned."""
        frame = np.ascontiguousarray(frame, dtype=np.float32)
        if not (isinstance(out, np.ndarray) and out.dtype == np.float32 and out.flags["C_CONTIGUOUS"] and out.flags["WRITEABLE"]):
            raise capi.FynException(capi.ERR_INVALID, "the output buffer must be a writable C-contiguous float32 array")
        n_in, n_out = getattr(self, "_async_sizes", (None, None))
        if n_in is None:
            raise capi.FynException(capi.ERR_STATE, "no frame pipeline is active")
        if frame.size != n_in or out.size != n_out:
            raise capi.FynException(capi.ERR_INVALID, "a frame takes %d floats in and %d out, the buffers hold %d and %d" % (n_in, n_out, frame.size, out.size))
        t = ctypes.c_uint64(0)
        capi.check(capi.lib().fyn_net_async_submit(self._h, capi.fptr(frame), capi.fptr(out), ctypes.byref(t)))
        self._async_outs[t.value] = out
        for old in [k for k in self._async_outs if k + 8 < t.value]:   # delivered when their slot was reused (depth <= 8)
            del self._async_outs[old]
        return t.value

    def asyncWait(self, ticket):
        capi.check(capi.lib().fyn_net_async_wait(self._h, ticket))
        for t in [k for k in self._async_outs if k <= ticket]:
            del self._async_outs[t]

    def asyncEnd(self):
        capi.check(capi.lib().fyn_net_async_end(self._h))
        self._async_outs = {}
        self._async_sizes = (None, None)

    def describe(self):
        """Plain description of the graph (descs, edges, loaded weight blocks) for external checkers."""
        out = []
        for lyr in self.layers:
            b = lyr.builder
            out.append({"builder": b, "number": lyr.number, "weights": lyr.weights})
        return {"layers": out, "connections": list(self.bufferManager.connections), "storage": self.storage}


class FramePool:
    """Several instances of one network, each with its own streams and frame pipeline.  Frames are dealt to the
    instances in turn, so that the kernels of up to `instances` frames share the GPU: small networks at batch 1 are
    bound by launch latency and leave most of the chip idle, and frames of different instances do not depend on each
    other.  Results are delivered in submission order through tickets, like NeuralNetwork.asyncSubmit / asyncWait
    (the reference runs one frame pipeline per network, base/engine.cpp:386-683; several of them side by side are
    several NeuralNetwork objects there as well).  More instances than hardware queues per process (4 by default)
    do not add throughput.

    make_net: callable returning a NeuralNetwork (not yet set up) with `input_key` and `output_layer` attributes.
    graph: replay each instance's forward pass as one captured graph, which cuts the host thread's share per frame from
    one launch per layer to one per frame (with 70-90 launches per frame the host thread is the limit otherwise)."""

    def __init__(self, make_net, instances=4, depth=2, inOrder=capi.ORDER_CHANNELWISE, outOrder=capi.ORDER_CHANNELWISE, graph=True):
        if instances < 1:
            raise capi.FynException(capi.ERR_INVALID, "a frame pool needs at least one network instance")
        self.nets, self._open, self._submitted = [], {}, 0
        try:
            for _ in range(instances):
                net = make_net()
                self.nets.append(net)
                net.setup()
                if graph:
                    net.useGraph(True)
                in_layer, in_port = net.input_key
                # one stream per instance: the instances overlap each other, and more streams than hardware queues
                # (4 per process by default) would wait for each other's events
                net.asyncBegin(in_layer, net.output_layer, inOrder, outOrder, depth, in_port, copyStreams=(instances == 1))
        except Exception:
            self.close()
            raise

    def submit(self, frame, out):
        """Queues one frame on the next instance; `out` is filled once wait(ticket) has returned.  Blocks while that
        instance's pipeline is full."""
        net = self.nets[self._submitted % len(self.nets)]
        self._submitted += 1
        self._open[self._submitted] = (net, net.asyncSubmit(frame, out))
        return self._submitted

    def wait(self, ticket):
        """Returns when the frame of `ticket` and every frame submitted before it have been delivered."""
        if ticket < 1 or ticket > self._submitted:
            raise capi.FynException(capi.ERR_INVALID, "unknown frame ticket %d" % ticket)
        for t in sorted(k for k in self._open if k <= ticket):
            net, local = self._open.pop(t)
            net.asyncWait(local)

    def close(self):
        for net in self.nets:
            try:
                net.asyncEnd()
            finally:
                net.cleanup()
        self.nets, self._open = [], {}
