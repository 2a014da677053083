"""Runtime: Device, Buffer, Graph over libmigemm.so.

The surface follows the reference runtime (/root/reference/vk.py:507-617 Buffer,
807-889 Graph, 892-1357 Device) for what the GEMM path uses.  What differs on a
discrete MI355X: host-visible kinds are pinned, device-mapped host memory (the
CPU view and the GPU pointer are the same bytes), "device" is HBM with no CPU
view, and all work runs on one in-order HIP stream instead of a Vulkan queue
with a barrier between dispatches.
"""

import ctypes as C
import time

import numpy as np

from . import _lib as L


class VkError(RuntimeError):
    """Any failure reported by the library (reference: vk.py:128-134)."""


def _check(rc, what=""):
    if rc != L.MG_OK:
        raise VkError(f"{what}: {L.last_error()} (code {rc})" if what else f"{L.last_error()} (code {rc})")


class Buffer:
    """GPU-visible memory of a kind.  If host-visible, .array() is a live numpy
    view of the bytes the GPU reads (vk.py:583-590)."""

    def __init__(self, dev, size, kind="shared"):
        if kind not in L.KINDS:
            raise VkError(f"unknown memory kind {kind!r}; use {list(L.KINDS)}")
        size = int(size)
        if size <= 0:
            raise VkError(f"buffer size must be positive, got {size}")
        self.dev, self.size, self.kind = dev, size, kind
        dptr, hptr = C.c_void_p(), C.c_void_p()
        _check(dev._lib.mg_alloc(dev._ctx, size, L.KINDS[kind], C.byref(dptr), C.byref(hptr)), "buffer")
        self.ptr = dptr.value           # device address
        self.host_ptr = hptr.value      # CPU address of the same bytes, or None
        self.host_visible = self.host_ptr is not None
        self.coherent = self.host_visible
        dev._buffers.add(self)

    def array(self, dtype, shape=None):
        if self.host_ptr is None:
            raise VkError(f"buffer kind={self.kind!r} is not host-visible")
        raw = (C.c_ubyte * self.size).from_address(self.host_ptr)
        a = np.frombuffer(raw, dtype=dtype)
        return a if shape is None else a.reshape(shape)

    def flush(self):
        """CPU writes -> visible to the GPU.  The mapping is coherent, so there
        is nothing to do (vk.py:592-598 is a no-op on coherent memory too)."""

    def invalidate(self):
        """GPU writes -> visible to the CPU: wait for the stream to drain."""
        if self.ptr is not None:
            _check(self.dev._lib.mg_sync(self.dev._ctx), "invalidate")

    def upload(self, arr):
        """Staged copy of a numpy array into this buffer (any kind)."""
        arr = np.ascontiguousarray(arr)
        if arr.nbytes > self.size:
            raise VkError(f"upload of {arr.nbytes} bytes into a buffer of {self.size}")
        _check(self.dev._lib.mg_upload(self.dev._ctx, self.ptr, arr.ctypes.data, arr.nbytes), "upload")

    def download(self, dtype, shape):
        """Staged copy of this buffer's leading bytes into a new numpy array."""
        out = np.empty(shape, dtype=dtype)
        if out.nbytes > self.size:
            raise VkError(f"download of {out.nbytes} bytes from a buffer of {self.size}")
        _check(self.dev._lib.mg_download(self.dev._ctx, out.ctypes.data, self.ptr, out.nbytes), "download")
        return out

    def destroy(self):
        if self.ptr is not None:
            ptr, self.ptr, self.host_ptr = self.ptr, None, None
            self.dev._buffers.discard(self)
            if self.dev._ctx is not None:
                _check(self.dev._lib.mg_free(self.dev._ctx, ptr, L.KINDS[self.kind]), "buffer destroy")


class Graph:
    """A recorded sequence of launches, replayed with one submit (vk.py:807-889).

    record() keeps each launch as a thunk; finish() captures them from the
    context's stream into a HIP graph; submit() replays it and waits.  Kernel
    arguments are baked in at finish(), so per-step values must live in buffers
    the CPU writes (same rule as the reference, vk.py:817-819)."""

    def __init__(self, dev, name="graph"):
        self.dev, self.name = dev, name
        self.n_dispatch = 0
        self._thunks = []
        self._finished = False
        self._handle = None
        self.traffic = []
        self.mm_split = []
        self._buffers = {}   # id -> every buffer a recorded launch names: its address is baked into the graph

    def record(self, launch, buffers=(), name="kernel", bytes_hint=None):
        """launch: zero-argument callable that enqueues work on the device
        stream (it must not synchronise)."""
        if self._finished:
            raise VkError(f"{self.name}: already finished")
        if not callable(launch):
            raise VkError(f"{self.name}: record() needs a callable launch")
        self._thunks.append(launch)
        for b in buffers:
            if b.ptr is None:
                raise VkError(f"{self.name}: {name} names a destroyed buffer")
            self._buffers[id(b)] = b
        compulsory = sum(b.size for b in buffers)
        self.traffic.append((name, compulsory, compulsory if bytes_hint is None else bytes_hint))
        self.n_dispatch += 1

    def fork(self):
        """From here on, launches recorded with side=True run on the device's side
        stream, after everything recorded so far and concurrently with what the main
        stream records next.  The reference puts a full barrier between any two
        dispatches (vk.py:848-851); independent products (dX and dW of a linear
        layer) need none."""
        if self._finished:
            raise VkError(f"{self.name}: already finished")
        self._thunks.append(self.dev.side_fork)

    def join(self):
        """Later main-stream launches wait for the side stream's work recorded so far
        (finish() joins by itself)."""
        if self._finished:
            raise VkError(f"{self.name}: already finished")
        self._thunks.append(self.dev.side_join)

    def finish(self):
        if self._finished:
            raise VkError(f"{self.name}: already finished")
        if not self._thunks:
            raise VkError(f"{self.name}: nothing recorded")
        lib, ctx = self.dev._lib, self.dev._ctx
        _check(lib.mg_graph_begin(ctx), f"{self.name}: finish")
        try:
            for t in self._thunks:
                t()
        except Exception:
            h = C.c_void_p()
            lib.mg_graph_end(ctx, C.byref(h))
            if h.value:
                lib.mg_graph_destroy(ctx, h)
            raise
        h = C.c_void_p()
        _check(lib.mg_graph_end(ctx, C.byref(h)), f"{self.name}: finish")
        self._handle = h
        self._finished = True
        self.dev._graphs.add(self)
        return self

    def _check_alive(self, what):
        """A finished graph holds raw device addresses: replaying it after one of its
        buffers was destroyed would run kernels on freed memory."""
        if not self._finished:
            raise VkError(f"{self.name}: call finish() before {what}()")
        if self._handle is None:
            raise VkError(f"{self.name}: {what}() on a destroyed graph")
        for b in self._buffers.values():
            if b.ptr is None:
                raise VkError(f"{self.name}: {what}() after a buffer of {b.size} bytes it uses was destroyed")

    def submit(self):
        self._check_alive("submit")
        dt = C.c_double()
        _check(self.dev._lib.mg_graph_launch(self.dev._ctx, self._handle, C.byref(dt)), f"{self.name}: submit")
        return dt.value

    def enqueue(self):
        """Replay without waiting; the stream keeps order with later work."""
        self._check_alive("enqueue")
        _check(self.dev._lib.mg_graph_enqueue(self.dev._ctx, self._handle), f"{self.name}: enqueue")

    def time(self, repeat=1):
        """Replay `repeat` times back to back; device seconds of each replay (HIP events
        on the context's stream)."""
        self._check_alive("time")
        out = (C.c_double * int(repeat))()
        _check(self.dev._lib.mg_graph_time(self.dev._ctx, self._handle, int(repeat), out), f"{self.name}: time")
        return list(out)

    def kernel_count(self):
        """Kernel launches one replay makes (a recorded call may stand for several)."""
        self._check_alive("kernel_count")
        n = C.c_int()
        _check(self.dev._lib.mg_graph_kernel_count(self.dev._ctx, self._handle, C.byref(n)), f"{self.name}: kernel_count")
        return n.value

    def destroy(self):
        if self._handle is not None:
            h, self._handle = self._handle, None
            self.dev._graphs.discard(self)
            if self.dev._ctx is not None:
                self.dev._lib.mg_graph_destroy(self.dev._ctx, h)


class Device:
    """One MI355X and one in-order stream (vk.py:892)."""

    KINDS = tuple(L.KINDS)

    def __init__(self, index=0):
        self._lib = L.load()
        ctx = C.c_void_p()
        rc = self._lib.mg_init(int(index), C.byref(ctx))
        self._ctx = None
        _check(rc, "Device")
        self._ctx = ctx
        self._buffers = set()
        self._graphs = set()
        info = L.DeviceInfo()
        _check(self._lib.mg_get_device_info(ctx, C.byref(info)), "Device")
        self.name = info.name.decode() or info.arch.decode()
        self.arch = info.arch.decode()
        self.compute_units = info.compute_units
        self.clock_khz = info.clock_khz
        self.total_mem = info.total_mem
        self.info = info
        # Attribute parity with the reference device (vk.py:1090-1120, 1128).
        self.has_coop_matrix = True
        self.subgroup_size_native = info.wavefront
        self.row_subgroup_size = info.wavefront

    def shader_core_props(self):
        """CU count and register file sizes (vk.py:1225-1240) for gfx950."""
        return dict(cus=self.compute_units, simd_per_cu=4, waves_per_simd=8,
                    wavefront_size=64, vgprs_per_simd=512, vgpr_granularity=8,
                    max_vgpr_alloc=512)

    def buffer(self, size, kind="shared"):
        return Buffer(self, size, kind)

    def graph(self, name="graph"):
        return Graph(self, name)

    def copy(self, src, dst, size=None, repeat=1):
        """Copy src -> dst on the device; returns wall seconds (vk.py:1267-1293)."""
        size = size if size is not None else min(src.size, dst.size)
        if size > src.size or size > dst.size:
            raise VkError(f"copy of {size} bytes exceeds a buffer ({src.size}, {dst.size})")
        t0 = time.perf_counter()
        for _ in range(repeat):
            _check(self._lib.mg_copy(self._ctx, dst.ptr, src.ptr, size), "copy")
        return time.perf_counter() - t0

    def side_fork(self):
        """The side stream waits for the main stream's work so far (mg_side_fork)."""
        _check(self._lib.mg_side_fork(self._ctx), "side_fork")

    def side_join(self):
        """The main stream waits for the side stream's work so far (mg_side_join)."""
        _check(self._lib.mg_side_join(self._ctx), "side_join")

    def sync(self):
        _check(self._lib.mg_sync(self._ctx), "sync")

    def destroy(self):
        if self._ctx is not None:
            for g in list(self._graphs):
                g.destroy()
            for b in list(self._buffers):
                b.destroy()
            ctx, self._ctx = self._ctx, None
            self._lib.mg_destroy(ctx)

    def __repr__(self):
        return (f"<Device {self.name!r} {self.arch} cus={self.compute_units} "
                f"clock={self.clock_khz / 1e6:.2f}GHz mem={self.total_mem / 2**30:.0f}GiB>")
