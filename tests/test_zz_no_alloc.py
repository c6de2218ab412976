"""The entry point that allocates nothing: l2_qlinear_matvec_device against l2_qlinear_matvec, through the
C ABI, on device buffers made with the HIP runtime directly (no torch)."""
import ctypes as C

import numpy as np
import pytest

from llama2_rs import checkpoint as ck

pytestmark = pytest.mark.gpu


class _Hip:
    """hipMalloc / hipMemcpy / hipDeviceSynchronize / hipFree through ctypes, for the test's own buffers."""

    def __init__(self):
        self.rt = C.CDLL("libamdhip64.so")
        self.rt.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        self.rt.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        self.rt.hipFree.argtypes = [C.c_void_p]
        self.rt.hipStreamCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.rt.hipStreamDestroy.argtypes = [C.c_void_p]
        self.rt.hipStreamSynchronize.argtypes = [C.c_void_p]
        self.rt.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
        self.rt.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        self.rt.hipGraphGetNodes.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_size_t)]
        self.rt.hipGraphNodeGetType.argtypes = [C.c_void_p, C.POINTER(C.c_int)]
        self.rt.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        self.rt.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
        self.rt.hipGraphExecDestroy.argtypes = [C.c_void_p]
        self.rt.hipGraphDestroy.argtypes = [C.c_void_p]
        self.bufs = []

    def upload(self, a: np.ndarray) -> int:
        p = C.c_void_p()
        assert self.rt.hipMalloc(C.byref(p), a.nbytes) == 0
        assert self.rt.hipMemcpy(p, a.ctypes.data_as(C.c_void_p), a.nbytes, 1) == 0   # host to device
        self.bufs.append(p)
        return p.value

    def empty(self, nbytes: int) -> int:
        p = C.c_void_p()
        assert self.rt.hipMalloc(C.byref(p), nbytes) == 0
        self.bufs.append(p)
        return p.value

    def download(self, p: int, shape) -> np.ndarray:
        out = np.empty(shape, np.float32)
        assert self.rt.hipDeviceSynchronize() == 0
        assert self.rt.hipMemcpy(out.ctypes.data_as(C.c_void_p), C.c_void_p(p), out.nbytes, 2) == 0   # device to host
        return out

    def close(self):
        for p in self.bufs:
            self.rt.hipFree(p)
        self.bufs = []


def test_matvec_without_allocation_equals_the_allocating_entry_point():
    from llama2_rs import ops, _lib
    from llama2_rs._lib import L2Error
    assert _lib.lib().l2_device_count() >= 1, "no HIP device: the GPU tests cannot run"
    hip = _Hip()
    rng = np.random.default_rng(0)
    big = ops.QLinear(*ck.synth_qlinear(rng, 4096, 1024, 128, act_order=True), 128)
    small = ops.QLinear(*ck.synth_qlinear(rng, 512, 264, 64, act_order=True), 64)
    # two calls in a row on the shared scratch, the second with a smaller input: the first fills 8 x 4096
    # floats of it, the second must not see any of them
    x1 = rng.standard_normal((8, 4096)).astype(np.float32)
    x2 = rng.standard_normal((3, 512)).astype(np.float32)
    x3 = rng.standard_normal((1, 4096)).astype(np.float32)
    want1, want2, want3 = big.matvec(x1), small.matvec(x2), big.matvec(x3)
    d1, d2, d3 = hip.upload(x1), hip.upload(x2), hip.upload(x3)
    y1, y2, y3 = hip.empty(want1.nbytes), hip.empty(want2.nbytes), hip.empty(want3.nbytes)
    big.matvec_device(d1, 8, y1)
    small.matvec_device(d2, 3, y2)
    big.matvec_device(d3, 1, y3)
    np.testing.assert_array_equal(hip.download(y1, want1.shape), want1)   # bit for bit
    np.testing.assert_array_equal(hip.download(y2, want2.shape), want2)
    np.testing.assert_array_equal(hip.download(y3, want3.shape), want3)
    # beyond the fixed scratch (2^20 floats): refused, nothing launched
    with pytest.raises(L2Error):
        big.matvec_device(d1, 257, y1)
    big.matvec_device(d1, 8, y1)
    np.testing.assert_array_equal(hip.download(y1, want1.shape), want1)
    big.close()
    small.close()
    hip.close()


def test_matvec_without_allocation_under_graph_capture():
    """The first call on a handle made while the stream is being captured (the handle's creation has done what a
    first launch does besides enqueueing), no memset node in the graph, and every replay — with eager work of the
    same operator and synchronisations between the replays — equal to the allocating entry point, bit for bit."""
    from llama2_rs import ops, _lib
    assert _lib.lib().l2_device_count() >= 1, "no HIP device: the GPU tests cannot run"
    hip = _Hip()
    rt = hip.rt
    rng = np.random.default_rng(1)
    q = ops.QLinear(*ck.synth_qlinear(rng, 4096, 512, 128, act_order=True), 128)
    other = ops.QLinear(*ck.synth_qlinear(rng, 1024, 264, 64, act_order=True), 64)
    xs = [rng.standard_normal((2, 4096)).astype(np.float32) for _ in range(3)]
    want = [q.matvec(x) for x in xs]
    dx, dy = hip.upload(xs[0]), hip.empty(want[0].nbytes)
    stream, graph, gexec = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert rt.hipStreamCreate(C.byref(stream)) == 0
    assert rt.hipStreamBeginCapture(stream, 0) == 0            # hipStreamCaptureModeGlobal
    try:
        q.matvec_device(dx, 2, dy, stream=stream.value)        # the handle's first device call: under capture
    finally:
        assert rt.hipStreamEndCapture(stream, C.byref(graph)) == 0
    n_nodes = C.c_size_t()
    assert rt.hipGraphGetNodes(graph, None, C.byref(n_nodes)) == 0 and n_nodes.value >= 2
    nodes = (C.c_void_p * n_nodes.value)()
    assert rt.hipGraphGetNodes(graph, nodes, C.byref(n_nodes)) == 0
    for node in nodes:
        kind = C.c_int()
        assert rt.hipGraphNodeGetType(C.c_void_p(node), C.byref(kind)) == 0
        assert kind.value == 0, f"graph node of type {kind.value}: only kernel nodes are expected"   # hipGraphNodeTypeKernel
    assert rt.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
    for x, w in zip(xs, want):
        assert rt.hipMemcpy(C.c_void_p(dx), x.ctypes.data_as(C.c_void_p), x.nbytes, 1) == 0
        assert rt.hipGraphLaunch(gexec, stream) == 0
        assert rt.hipStreamSynchronize(stream) == 0
        np.testing.assert_array_equal(hip.download(dy, w.shape), w)
        # eager work on the shared scratch between the replays
        x2 = rng.standard_normal((3, 1024)).astype(np.float32)
        d2, y2 = hip.upload(x2), hip.empty(3 * 264 * 4)
        other.matvec_device(d2, 3, y2)
        np.testing.assert_array_equal(hip.download(y2, (3, 264)), other.matvec(x2))
    assert rt.hipGraphExecDestroy(gexec) == 0
    assert rt.hipGraphDestroy(graph) == 0
    assert rt.hipStreamDestroy(stream) == 0
    q.close()
    other.close()
    hip.close()
