"""rd_topk_rows_static — the top-K of logits rows with nothing allocated (static device scratch, device pointers in and out) —
against rd_topk_rows on the same rows: ids, logit bits and Z identical, on two calls in a row, the second smaller than the first
(so the second call meets the first call's leftovers in the shared scratch)."""
import ctypes as C

import numpy as np
import pytest

from goinfer_amd import capi

pytestmark = pytest.mark.gpu


class Hip:
    """Just enough of the HIP runtime, through ctypes, for a test to own device buffers."""

    def __init__(self):
        self.lib = C.CDLL("libamdhip64.so.7")
        self.bufs = []

    def check(self, rc, what):
        assert rc == 0, "%s failed (%d)" % (what, rc)

    def to_device(self, a):
        a = np.ascontiguousarray(a)
        p = self.alloc(a.nbytes)
        self.check(self.lib.hipMemcpy(p, a.ctypes.data_as(C.c_void_p), C.c_size_t(a.nbytes), 1), "hipMemcpy H2D")
        return p

    def alloc(self, nbytes):
        p = C.c_void_p()
        self.check(self.lib.hipMalloc(C.byref(p), C.c_size_t(max(nbytes, 16))), "hipMalloc")
        self.bufs.append(p)
        return p

    def to_host(self, p, shape, dtype):
        out = np.empty(shape, dtype)
        self.check(self.lib.hipDeviceSynchronize(), "hipDeviceSynchronize")
        self.check(self.lib.hipMemcpy(out.ctypes.data_as(C.c_void_p), p, C.c_size_t(out.nbytes), 2), "hipMemcpy D2H")
        return out

    def free_all(self):
        for p in self.bufs:
            self.lib.hipFree(p)
        self.bufs = []


def bell_rows(rows, V, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((rows, V)).astype(np.float32) * 2.5
    x[:, ::97] = np.float32(1.25)  # ties, broken by token id
    return x


def static_topk(hip, x, k, T, want_z=True):
    rows, V = x.shape
    kk = min(k, V)
    dl = hip.to_device(x)
    di, dv, dz = hip.alloc(rows * kk * 4), hip.alloc(rows * kk * 4), hip.alloc(rows * 8)
    capi.check(capi.lib().rd_topk_rows_static(0, None, dl, rows, V, k, C.c_double(T), int(want_z), di, dv, dz if want_z else None), "rd_topk_rows_static")
    ids, vals = hip.to_host(di, (rows, kk), np.int32), hip.to_host(dv, (rows, kk), np.float32)
    z = hip.to_host(dz, (rows,), np.float64) if want_z else None
    return ids, vals, z


def test_static_scratch_topk_equals_the_allocating_entry_point():
    dev = capi.Device(0)
    hip = Hip()
    try:
        # first call: as wide and as many rows as the step's top-K sees; second call: fewer, narrower rows and another k
        for rows, V, k, T in ((32, 128256, 256, 0.7), (5, 40000, 50, 1.3), (3, 5000, 17, 1.0)):
            x = bell_rows(rows, V, 11 + rows)
            wi, wv, wz = dev.topk_rows(x, k, T)
            gi, gv, gz = static_topk(hip, x, k, T)
            assert np.array_equal(gi, wi), (rows, V, k)
            assert np.array_equal(gv.view(np.uint32), wv.view(np.uint32)), (rows, V, k)
            assert np.array_equal(gz, wz), (rows, V, k)
        # without Z
        x = bell_rows(4, 70000, 3)
        wi, wv, _ = dev.topk_rows(x, 1024, 1.0, want_z=False)
        gi, gv, _ = static_topk(hip, x, 1024, 1.0, want_z=False)
        assert np.array_equal(gi, wi) and np.array_equal(gv.view(np.uint32), wv.view(np.uint32))
    finally:
        hip.free_all()
        dev.close()


def test_static_scratch_topk_rejects_what_exceeds_its_scratch():
    dev = capi.Device(0)
    hip = Hip()
    try:
        p = hip.alloc(64)
        L = capi.lib()
        for rows, V, k in ((33, 1000, 4), (1, 262145, 4), (1, 1000, 0), (1, 1000, 1025), (0, 1000, 4)):
            rc = L.rd_topk_rows_static(0, None, p, rows, V, k, C.c_double(1.0), 0, p, p, None)
            assert rc == -1, (rows, V, k, rc)
            assert b"rd_topk_rows_static" in L.rd_last_error()
        assert L.rd_topk_rows_static(0, None, None, 1, 1000, 4, C.c_double(1.0), 0, p, p, None) == -1
    finally:
        hip.free_all()
        dev.close()


def test_static_scratch_topk_under_stream_capture():
    """What the entry point is for: captured on a caller-owned stream into a graph (the device was opened before, so nothing is left
    to set up), replayed on fresh logits in the same buffers with ordinary work in between; every replay equals rd_topk_rows on the
    same rows, bit for bit. An error left behind by an unrelated earlier call is not reported as this call's."""
    dev = capi.Device(0)
    hip = Hip()
    L = hip.lib
    try:
        rows, V, k, T = 8, 151936, 256, 0.8
        dl = hip.alloc(rows * V * 4)
        di, dv, dz = hip.alloc(rows * k * 4), hip.alloc(rows * k * 4), hip.alloc(rows * 8)
        stream, graph, gexec = C.c_void_p(), C.c_void_p(), C.c_void_p()
        hip.check(L.hipStreamCreate(C.byref(stream)), "hipStreamCreate")
        assert L.hipFree(C.c_void_p(16)) != 0  # leaves a sticky-until-read error behind
        hip.check(L.hipStreamBeginCapture(stream, 1), "hipStreamBeginCapture")  # 1 = hipStreamCaptureModeThreadLocal
        rc = capi.lib().rd_topk_rows_static(0, stream, dl, rows, V, k, C.c_double(T), 1, di, dv, dz)
        end = L.hipStreamEndCapture(stream, C.byref(graph))
        capi.check(rc, "rd_topk_rows_static under capture")
        hip.check(end, "hipStreamEndCapture")
        hip.check(L.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)), "hipGraphInstantiate")
        for rep in range(3):
            x = bell_rows(rows, V, 100 + rep)
            hip.check(L.hipMemcpy(dl, x.ctypes.data_as(C.c_void_p), C.c_size_t(x.nbytes), 1), "hipMemcpy H2D")
            wi, wv, wz = dev.topk_rows(x, k, T)  # the program's own eager work between the replays
            hip.check(L.hipGraphLaunch(gexec, stream), "hipGraphLaunch")
            hip.check(L.hipStreamSynchronize(stream), "hipStreamSynchronize")
            gi, gv, gz = hip.to_host(di, (rows, k), np.int32), hip.to_host(dv, (rows, k), np.float32), hip.to_host(dz, (rows,), np.float64)
            assert np.array_equal(gi, wi), rep
            assert np.array_equal(gv.view(np.uint32), wv.view(np.uint32)), rep
            assert np.array_equal(gz, wz), rep
        hip.check(L.hipGraphExecDestroy(gexec), "hipGraphExecDestroy")
        hip.check(L.hipGraphDestroy(graph), "hipGraphDestroy")
        hip.check(L.hipStreamDestroy(stream), "hipStreamDestroy")
    finally:
        hip.free_all()
        dev.close()
