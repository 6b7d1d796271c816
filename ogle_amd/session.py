"""ctypes binding of the graph runtime's C ABI (include/ogle_runtime.h).

`Session` mirrors opengl::FBOSession (ogl_runtime/opengl/core/fbo_session.h:11-90):
load_graph, run, get_outputs, plus the additions of this runtime (compute with
resident inputs, hipGraph replay, per-node timing) and the SSD Detector.
"""
import ctypes
import os

import numpy as np

from . import hip as _hip

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libogle_runtime.so")

SYMBOLS = [
    "ogle_rt_last_error", "ogle_rt_session_create", "ogle_rt_session_destroy",
    "ogle_rt_load_file", "ogle_rt_load_bytes", "ogle_rt_run", "ogle_rt_compute",
    "ogle_rt_compute_graph", "ogle_rt_sync", "ogle_rt_time_compute", "ogle_rt_profile",
    "ogle_rt_profile_entry", "ogle_rt_tensor_shape", "ogle_rt_tensor_device_ptr",
    "ogle_rt_time_pipelined", "ogle_rt_alloc_pinned", "ogle_rt_free_pinned",
    "ogle_rt_stream", "ogle_rt_get_output", "ogle_rt_num_kernels",
    "ogle_rt_registered_kernel_count", "ogle_rt_registered_kernel_name", "ogle_rt_detect",
    "ogle_rt_reserialize", "ogle_rt_model_debug_string", "ogle_rt_tensor_dformat",
    "ogle_rt_set_reorder", "ogle_rt_issue_order_name", "ogle_rt_set_device_nms",
    "ogle_rt_detect_results", "ogle_rt_graph_captured", "ogle_rt_hazard_conflicts",
    "ogle_rt_set_fuse_siblings", "ogle_rt_launch_plan", "ogle_rt_launch_plan_entry",
    "ogle_rt_conv_hazard_conflicts", "ogle_rt_host_elements", "ogle_rt_time_pipelined_readback",
    "ogle_rt_pipelined_results",
]


class Detection(ctypes.Structure):
    _fields_ = [("image", ctypes.c_int32), ("prior", ctypes.c_int32), ("class_id", ctypes.c_int32),
                ("score", ctypes.c_float), ("x", ctypes.c_int32), ("y", ctypes.c_int32),
                ("width", ctypes.c_int32), ("height", ctypes.c_int32), ("cx", ctypes.c_float),
                ("cy", ctypes.c_float)]


class RuntimeError_(RuntimeError):
    pass


_lib = None


def lib():
    global _lib
    if _lib is None:
        _hip.lib()  # the kernels first: fails loudly if they were not built
        if not os.path.exists(LIB_PATH):
            raise RuntimeError_("%s is missing: build it with `make -C ogle_amd/runtime`" % LIB_PATH)
        l = ctypes.CDLL(LIB_PATH)
        vp, i32, i64, cp = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_char_p
        l.ogle_rt_last_error.restype = cp
        l.ogle_rt_session_create.restype = vp
        l.ogle_rt_session_destroy.argtypes = [vp]
        l.ogle_rt_load_file.argtypes = [vp, cp]
        l.ogle_rt_load_bytes.argtypes = [vp, vp, ctypes.c_size_t]
        l.ogle_rt_run.argtypes = [vp, i32, ctypes.POINTER(cp), ctypes.POINTER(vp),
                                  ctypes.POINTER(ctypes.POINTER(i32)), ctypes.POINTER(i32),
                                  ctypes.POINTER(cp)]
        l.ogle_rt_host_elements.argtypes = [ctypes.POINTER(i32), i32, cp]
        l.ogle_rt_host_elements.restype = i64
        l.ogle_rt_compute.argtypes = [vp]
        l.ogle_rt_compute_graph.argtypes = [vp]
        l.ogle_rt_sync.argtypes = [vp]
        l.ogle_rt_graph_captured.argtypes = [vp, i32]
        l.ogle_rt_hazard_conflicts.argtypes = [
            ctypes.POINTER(_hip.ConvArgs), i32, ctypes.POINTER(vp), ctypes.POINTER(ctypes.c_size_t),
            i32, ctypes.POINTER(vp), ctypes.POINTER(ctypes.c_size_t), i32]
        l.ogle_rt_conv_hazard_conflicts.argtypes = [ctypes.POINTER(_hip.ConvArgs), i32,
                                                    ctypes.POINTER(_hip.ConvArgs)]
        l.ogle_rt_time_compute.argtypes = [vp, i32, i32, i32, i32, i32,
                                           ctypes.POINTER(ctypes.c_float),
                                           ctypes.POINTER(ctypes.c_float)]
        l.ogle_rt_time_pipelined.argtypes = [ctypes.POINTER(vp), i32, i32, i32, i32, cp,
                                             ctypes.POINTER(vp), ctypes.POINTER(ctypes.c_float)]
        l.ogle_rt_alloc_pinned.argtypes = [ctypes.c_size_t]
        l.ogle_rt_alloc_pinned.restype = vp
        l.ogle_rt_free_pinned.argtypes = [vp]
        l.ogle_rt_free_pinned.restype = None
        l.ogle_rt_profile.argtypes = [vp]
        l.ogle_rt_launch_plan.argtypes = [vp, i32]
        l.ogle_rt_launch_plan_entry.argtypes = [vp, i32, ctypes.POINTER(cp), ctypes.POINTER(i32),
                                                ctypes.POINTER(ctypes.c_float), i32]
        l.ogle_rt_profile_entry.argtypes = [vp, i32, ctypes.POINTER(cp), ctypes.POINTER(cp),
                                            ctypes.POINTER(ctypes.c_float)]
        l.ogle_rt_tensor_shape.argtypes = [vp, cp, ctypes.POINTER(i32)]
        l.ogle_rt_tensor_dformat.argtypes = [vp, cp]
        l.ogle_rt_tensor_device_ptr.argtypes = [vp, cp]
        l.ogle_rt_tensor_device_ptr.restype = vp
        l.ogle_rt_stream.argtypes = [vp]
        l.ogle_rt_stream.restype = vp
        l.ogle_rt_get_output.argtypes = [vp, cp, cp, vp, i64]
        l.ogle_rt_get_output.restype = i64
        l.ogle_rt_num_kernels.argtypes = [vp]
        l.ogle_rt_set_reorder.argtypes = [vp, i32]
        l.ogle_rt_set_fuse_siblings.argtypes = [vp, i32]
        l.ogle_rt_set_device_nms.argtypes = [vp, i32]
        l.ogle_rt_issue_order_name.argtypes = [vp, i32]
        l.ogle_rt_issue_order_name.restype = cp
        l.ogle_rt_registered_kernel_name.argtypes = [i32]
        l.ogle_rt_registered_kernel_name.restype = cp
        l.ogle_rt_detect.argtypes = [vp, vp, ctypes.POINTER(i32), cp, cp, cp, cp, ctypes.c_float,
                                     ctypes.c_float, i32, i32, i32, ctypes.POINTER(Detection), i64]
        l.ogle_rt_detect.restype = i64
        l.ogle_rt_detect_results.argtypes = [vp, ctypes.POINTER(Detection), i64]
        l.ogle_rt_detect_results.restype = i64
        l.ogle_rt_time_pipelined_readback.argtypes = [ctypes.POINTER(vp), i32, i32, i32,
                                                      ctypes.POINTER(ctypes.c_float), ctypes.POINTER(i64)]
        l.ogle_rt_pipelined_results.argtypes = [vp, ctypes.POINTER(Detection), i64]
        l.ogle_rt_pipelined_results.restype = i64
        l.ogle_rt_reserialize.argtypes = [vp, ctypes.c_size_t, vp, i64]
        l.ogle_rt_reserialize.restype = i64
        l.ogle_rt_model_debug_string.argtypes = [vp, ctypes.c_size_t, vp, i64]
        l.ogle_rt_model_debug_string.restype = i64
        _lib = l
    return _lib


def _check(rc):
    if rc < 0:
        raise RuntimeError_(lib().ogle_rt_last_error().decode())
    return rc


def reserialize(model_bytes):
    """Round trip through the runtime's C++ .dlx codec (parse, then serialize)."""
    src = ctypes.create_string_buffer(bytes(model_bytes), len(model_bytes))
    dst = ctypes.create_string_buffer(len(model_bytes) + 1024)
    n = _check(lib().ogle_rt_reserialize(ctypes.cast(src, ctypes.c_void_p), len(model_bytes),
                                         ctypes.cast(dst, ctypes.c_void_p), len(dst)))
    return dst.raw[:n]


def model_debug_string(model_bytes):
    src = ctypes.create_string_buffer(bytes(model_bytes), len(model_bytes))
    dst = ctypes.create_string_buffer(1 << 22)
    _check(lib().ogle_rt_model_debug_string(ctypes.cast(src, ctypes.c_void_p), len(model_bytes),
                                            ctypes.cast(dst, ctypes.c_void_p), len(dst)))
    return dst.value.decode()


def hazard_conflicts(pending, reads, writes):
    """The executor's dependency rule on plain numbers (no device): `pending` is a list of
    hip.ConvArgs (deferred convolutions), `reads` / `writes` lists of (address, bytes).
    True if the launch must wait for one of them."""
    arr = (_hip.ConvArgs * max(1, len(pending)))(*pending)

    def split(ranges):
        n = max(1, len(ranges))
        ptrs = (ctypes.c_void_p * n)(*[r[0] for r in ranges])
        sizes = (ctypes.c_size_t * n)(*[r[1] for r in ranges])
        return ptrs, sizes
    rp, rb = split(reads)
    wp, wb = split(writes)
    return bool(_check(lib().ogle_rt_hazard_conflicts(arr, len(pending), rp, rb, len(reads), wp, wb,
                                                      len(writes))))


def conv_hazard_conflicts(pending, nxt):
    """The same rule with a convolution (hip.ConvArgs) as the next launch."""
    arr = (_hip.ConvArgs * max(1, len(pending)))(*pending)
    return bool(_check(lib().ogle_rt_conv_hazard_conflicts(arr, len(pending), ctypes.byref(nxt))))


def registered_kernels():
    l = lib()
    return [l.ogle_rt_registered_kernel_name(i).decode()
            for i in range(l.ogle_rt_registered_kernel_count())]


class PinnedBuffer:
    """Page-locked host memory (ogle_rt_alloc_pinned) viewed as a numpy array."""

    def __init__(self, shape, dtype=np.float32):
        self.nbytes = int(np.prod(shape)) * np.dtype(dtype).itemsize
        self.ptr = lib().ogle_rt_alloc_pinned(self.nbytes)
        if not self.ptr:
            raise MemoryError("ogle_rt_alloc_pinned(%d) failed" % self.nbytes)
        buf = (ctypes.c_char * self.nbytes).from_address(self.ptr)
        self.array = np.frombuffer(buf, dtype=dtype).reshape(shape)

    def close(self):
        if self.ptr:
            self.array = None
            lib().ogle_rt_free_pinned(self.ptr)
            self.ptr = None

    def __del__(self):
        self.close()


def host_elements(shape, dformat):
    """Floats a host buffer of logical shape `shape` holds in layout `dformat` (the dense
    product for NHWC / NCHW / ANY, the stride-4 padded sizes for NHWC4 / ANY4 / HWN4C4)."""
    dims = (ctypes.c_int32 * max(len(shape), 1))(*shape)
    return _check(lib().ogle_rt_host_elements(dims, len(shape), dformat.encode()))


class Session:
    def __init__(self):
        self._h = lib().ogle_rt_session_create()
        if not self._h:
            raise RuntimeError_(lib().ogle_rt_last_error().decode())

    def close(self):
        if self._h:
            lib().ogle_rt_session_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def load_graph(self, model):
        """model: a path, serialized bytes, or a dlx.GraphBuilder."""
        if hasattr(model, "serialize"):
            model = model.serialize()
        if isinstance(model, (bytes, bytearray)):
            buf = ctypes.create_string_buffer(bytes(model), len(model))
            _check(lib().ogle_rt_load_bytes(self._h, ctypes.cast(buf, ctypes.c_void_p), len(model)))
        else:
            _check(lib().ogle_rt_load_file(self._h, str(model).encode()))

    def run(self, inputs, dformats=None, shapes=None):
        """inputs: {name: float32 ndarray}; dformats: {name: "NHWC"|"NCHW"|"ANY"} (default NHWC
        for rank 4, ANY otherwise).  An input in one of the padded layouts ("NHWC4", "ANY4")
        also needs its logical shape in `shapes`."""
        names = list(inputs)
        arrs = [np.ascontiguousarray(inputs[n], dtype=np.float32) for n in names]
        n = len(names)
        c_names = (ctypes.c_char_p * n)(*[s.encode() for s in names])
        c_data = (ctypes.c_void_p * n)(*[a.ctypes.data for a in arrs])
        logical = [tuple((shapes or {}).get(nm, a.shape)) for nm, a in zip(names, arrs)]
        dims = [(ctypes.c_int32 * len(sh))(*sh) for sh in logical]
        c_dims = (ctypes.POINTER(ctypes.c_int32) * n)(
            *[ctypes.cast(d, ctypes.POINTER(ctypes.c_int32)) for d in dims])
        c_ranks = (ctypes.c_int32 * n)(*[len(sh) for sh in logical])
        fm = [(dformats or {}).get(nm, "NHWC" if a.ndim == 4 else "ANY") for nm, a in zip(names, arrs)]
        c_fm = (ctypes.c_char_p * n)(*[f.encode() for f in fm])
        # the runtime reads host_elements(logical shape, tag) floats from each buffer: a dense
        # array under a padded tag (or any other size mismatch) would be read past its end
        for nm, a, d, sh, f in zip(names, arrs, dims, logical, fm):
            need = host_elements(sh, f)
            if a.size != need:
                raise ValueError("input %r: layout %s of logical shape %s takes %d floats, the array "
                                 "holds %d%s" % (nm, f, sh, need, a.size,
                                                 "" if (shapes or {}).get(nm) is not None or not f.endswith("4")
                                                 else " (pass the logical shape in `shapes`)"))
        _check(lib().ogle_rt_run(self._h, n, c_names, c_data, c_dims, c_ranks, c_fm))

    def compute(self, graph=False):
        _check(lib().ogle_rt_compute_graph(self._h) if graph else lib().ogle_rt_compute(self._h))

    def graph_captured(self, slot=0):
        return bool(_check(lib().ogle_rt_graph_captured(self._h, slot)))

    def sync(self):
        _check(lib().ogle_rt_sync(self._h))

    def time_compute(self, warmup, iters, graph=False, with_detect=False, sync_each=False):
        """Returns (per-pass ms array, total ms) measured with HIP events on the session stream.
        with_detect appends the SSD decode + score-filter launch to every pass; sync_each waits
        for each pass before the next is enqueued (per-pass latency instead of throughput)."""
        each = (ctypes.c_float * iters)()
        total = ctypes.c_float(0)
        _check(lib().ogle_rt_time_compute(self._h, warmup, iters, 1 if graph else 0,
                                          1 if with_detect else 0, 1 if sync_each else 0, each,
                                          ctypes.byref(total)))
        return np.array(each[:], np.float64), float(total.value)

    @staticmethod
    def time_pipelined(sessions, warmup, iters, with_detect=True, input_name=None, host_inputs=None):
        """`iters` passes dealt round-robin over `sessions` (same graph), each replaying its
        hipGraph on its own stream.  With `host_inputs` (one PinnedBuffer per session holding the
        bytes of input `input_name`) every pass first copies its input to the device on its
        stream; otherwise the inputs stay resident.  Returns the total ms from a common idle start
        until every stream is idle again."""
        handles = (ctypes.c_void_p * len(sessions))(*[s._h for s in sessions])
        total = ctypes.c_float(0)
        hosts = None
        if host_inputs is not None:
            assert input_name is not None and len(host_inputs) == len(sessions)
            hosts = (ctypes.c_void_p * len(sessions))(*[h.ptr for h in host_inputs])
        _check(lib().ogle_rt_time_pipelined(handles, len(sessions), warmup, iters,
                                            1 if with_detect else 0,
                                            input_name.encode() if input_name else None, hosts,
                                            ctypes.byref(total)))
        return float(total.value)

    def profile(self):
        """One pass with per-node events: list of (label, type, ms)."""
        n = _check(lib().ogle_rt_profile(self._h))
        out = []
        label, typ, ms = ctypes.c_char_p(), ctypes.c_char_p(), ctypes.c_float()
        for i in range(n):
            _check(lib().ogle_rt_profile_entry(self._h, i, ctypes.byref(label), ctypes.byref(typ),
                                               ctypes.byref(ms)))
            out.append((label.value.decode(), typ.value.decode(), float(ms.value)))
        return out

    def launch_plan(self, with_detect=False, durations=False):
        """Dispatch sequence of one (eager) pass: list of (label, dispatches) in issue order; a
        label is "<node>#<type>#", several joined with '+' for convolutions that share grids.
        With durations=True each entry is (label, [microseconds per device operation]), the
        kernels' own device-stamped durations in that pass."""
        n = _check(lib().ogle_rt_launch_plan(self._h, 1 if with_detect else 0))
        out = []
        label, k = ctypes.c_char_p(), ctypes.c_int32()
        cap = 64
        us = (ctypes.c_float * cap)()
        for i in range(n):
            _check(lib().ogle_rt_launch_plan_entry(self._h, i, ctypes.byref(label), ctypes.byref(k), us, cap))
            if k.value > cap:  # an entry with more device operations than the buffer: read it again
                cap = k.value
                us = (ctypes.c_float * cap)()
                _check(lib().ogle_rt_launch_plan_entry(self._h, i, ctypes.byref(label), ctypes.byref(k), us, cap))
            out.append((label.value.decode(), [float(v) for v in us[:k.value]] if durations else int(k.value)))
        return out

    def tensor_shape(self, name):
        dims = (ctypes.c_int32 * 8)()
        rank = _check(lib().ogle_rt_tensor_shape(self._h, name.encode(), dims))
        return tuple(dims[:rank])

    def tensor_dformat(self, name):
        """Layout tag as a string: "NHWC4", "ANY4", "HWN4C4", ..."""
        from . import dlx
        return dlx.DFORMAT_NAMES[_check(lib().ogle_rt_tensor_dformat(self._h, name.encode()))]

    def tensor_device_ptr(self, name):
        return lib().ogle_rt_tensor_device_ptr(self._h, name.encode())

    @property
    def stream(self):
        return lib().ogle_rt_stream(self._h)

    @property
    def num_kernels(self):
        return lib().ogle_rt_num_kernels(self._h)

    def set_device_nms(self, on):
        """Top-k + NMS of detect() on the device (default) or on the host."""
        _check(lib().ogle_rt_set_device_nms(self._h, 1 if on else 0))

    def set_reorder(self, on):
        """Before the first run: False keeps the reference's strict file order."""
        _check(lib().ogle_rt_set_reorder(self._h, 1 if on else 0))

    def set_fuse_siblings(self, on):
        """Before the first run: True runs Conv nodes that read the same tensor with the same
        attributes (an SSD feature map's box and class head) as one launch."""
        _check(lib().ogle_rt_set_fuse_siblings(self._h, 1 if on else 0))

    def issue_order(self):
        """Node names in the order a pass issues them (after the first run)."""
        names, i = [], 0
        while True:
            p = lib().ogle_rt_issue_order_name(self._h, i)
            if p is None:
                return names
            names.append(p.decode())
            i += 1

    def get_output(self, name, dformat="ANY"):
        shape = self.tensor_shape(name)
        out = np.empty(shape, np.float32)
        up4 = lambda v: (v + 3) // 4 * 4
        if dformat in ("NHWC4", "ANY4") and len(shape) > 0:
            # the reference's padded host layouts: last dimension padded to a multiple of 4
            out = np.empty(tuple(shape[:-1]) + (up4(shape[-1]),), np.float32)
        elif dformat == "HWN4C4" and len(shape) == 4:
            o, i, kh, kw = shape  # an OIHW filter: (kh*kw*ceil(O/4), ceil(I/4)*4, 4) texels
            out = np.empty((kh * kw * ((o + 3) // 4), up4(i), 4), np.float32)
        if dformat == "NCHW" and len(shape) == 4 and self.tensor_dformat(name) in ("NHWC", "NHWC4"):
            out = np.empty((shape[0], shape[3], shape[1], shape[2]), np.float32)
        n = _check(lib().ogle_rt_get_output(self._h, name.encode(), dformat.encode(),
                                            out.ctypes.data, out.size))
        assert n == out.size
        return out

    def get_outputs(self, names, dformats):
        return [self.get_output(n, f) for n, f in zip(names, dformats)]

    def detect(self, images, raw_width, raw_height, score_threshold=0.3, nms_threshold=0.45,
               topk=100, input_name=None, output_names=None, capacity=4096):
        images = np.ascontiguousarray(images, dtype=np.float32)
        dims = (ctypes.c_int32 * 4)(*images.shape)
        names = [None, None, None] if output_names is None else [s.encode() for s in output_names]
        buf = (Detection * capacity)()
        n = _check(lib().ogle_rt_detect(self._h, images.ctypes.data, dims,
                                        input_name.encode() if input_name else None, names[0],
                                        names[1], names[2], score_threshold, nms_threshold, topk,
                                        raw_width, raw_height, buf, capacity))
        return self._per_image(buf, n, capacity, images.shape[0])

    @staticmethod
    def _per_image(buf, n, capacity, batch):
        per_image = [[] for _ in range(batch)]
        for d in buf[:min(n, capacity)]:
            per_image[d.image].append(dict(prior=d.prior, cls=d.class_id, score=d.score,
                                           rect=(d.x, d.y, d.width, d.height), cx=d.cx, cy=d.cy))
        return per_image

    @staticmethod
    def time_pipelined_readback(sessions, warmup, iters):
        """`iters` passes dealt round-robin over `sessions`, each pass a hipGraph replay on its
        session's stream that ends with one asynchronous copy of its final detection lists to
        page-locked host memory; before a session's next pass is launched the host waits for the
        event behind its previous pass and reads the lists.  Returns (total ms, detections read
        in the timed passes)."""
        handles = (ctypes.c_void_p * len(sessions))(*[s._h for s in sessions])
        total, seen = ctypes.c_float(0), ctypes.c_int64(0)
        _check(lib().ogle_rt_time_pipelined_readback(handles, len(sessions), warmup, iters,
                                                     ctypes.byref(total), ctypes.byref(seen)))
        return float(total.value), int(seen.value)

    def pipelined_results(self, batch, capacity=4096):
        """Detections of the session's last pass of time_pipelined_readback, from the page-locked
        copy of its lists."""
        buf = (Detection * capacity)()
        n = _check(lib().ogle_rt_pipelined_results(self._h, buf, capacity))
        return self._per_image(buf, n, capacity, batch)

    def detect_results(self, batch, capacity=4096):
        """Detections of the detector work last enqueued by time_compute(with_detect=True)."""
        buf = (Detection * capacity)()
        n = _check(lib().ogle_rt_detect_results(self._h, buf, capacity))
        return self._per_image(buf, n, capacity, batch)
