"""ctypes binding of libskm_hip.so (the C ABI declared in include/skm_hip.h).

This is plumbing for tests, the benchmark and the Python facade: every compute call goes to the
HIP library; there is no CPU fallback.  Loading fails loudly when the library has not been built.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_double, c_float, c_int, c_size_t, c_uint32, c_uint64, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libskm_hip.so")

_F = c_void_p  # device pointers travel as opaque addresses


class SkmError(RuntimeError):
    pass


_PROTOTYPES = {
    "skm_last_error": (c_char_p, []),
    "skm_device_count": (c_int, [POINTER(c_int)]),
    "skm_ctx_create": (c_int, [c_int, POINTER(c_void_p)]),
    "skm_ctx_destroy": (c_int, [c_void_p]),
    "skm_sync": (c_int, [c_void_p]),
    "skm_ctx_set_workspace_limit": (c_int, [c_void_p, c_size_t]),
    "skm_malloc": (c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    "skm_free": (c_int, [c_void_p, c_void_p]),
    "skm_upload": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "skm_download": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "skm_copy": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "skm_fill_u32": (c_int, [c_void_p, c_void_p, c_uint32, c_size_t]),
    "skm_prof_enable": (c_int, [c_void_p, c_int]),
    "skm_prof_reset": (c_int, [c_void_p]),
    "skm_prof_get": (c_int, [c_void_p, c_char_p, POINTER(c_double), POINTER(c_uint64)]),
    "skm_prof_dump": (c_int, [c_void_p, c_char_p, c_size_t, POINTER(c_size_t)]),
    "skm_norms": (c_int, [c_void_p, _F, c_size_t, c_size_t, c_size_t, _F]),
    "skm_rotate": (c_int, [c_void_p, _F, c_size_t, c_size_t, _F, _F]),
    "skm_unrotate": (c_int, [c_void_p, _F, c_size_t, c_size_t, _F, _F]),
    "skm_transpose": (c_int, [c_void_p, _F, c_size_t, c_size_t, _F]),
    "skm_pdxify": (c_int, [c_void_p, _F, c_size_t, c_size_t, c_size_t, _F, _F]),
    "skm_assign_full": (c_int, [c_void_p, _F, c_size_t, _F, c_size_t, c_size_t, _F, _F, _F, _F]),
    "skm_assign_pruned": (
        c_int,
        [c_void_p, _F, c_size_t, _F, _F, _F, c_size_t, c_size_t, c_size_t, c_uint32, _F, _F, _F, _F, _F,
         POINTER(c_uint64), POINTER(c_uint64)],
    ),
    "skm_update": (c_int, [c_void_p, _F, c_size_t, c_size_t, _F, c_size_t, _F, _F]),
    "skm_scale_by_size": (c_int, [c_void_p, _F, _F, c_size_t, c_size_t]),
    "skm_normalize_rows": (c_int, [c_void_p, _F, c_size_t, c_size_t]),
    "skm_edit_rows": (c_int, [c_void_p, _F, c_size_t, c_void_p, c_size_t]),
    "skm_wcss": (c_int, [c_void_p, _F, c_size_t, POINTER(c_double)]),
    "skm_shift": (c_int, [c_void_p, _F, _F, c_size_t, c_size_t, POINTER(c_double)]),
    "skm_gather_rows": (c_int, [c_void_p, _F, c_size_t, _F, c_size_t, _F, _F, _F]),
    "skm_scatter_assignments": (c_int, [c_void_p, _F, _F, c_size_t, c_uint32, _F]),
}

_lib = None


def exported_symbols():
    """Names every build of the library must export (mirrors include/skm_hip.h)."""
    return sorted(_PROTOTYPES)


def load():
    """Loads libskm_hip.so and attaches prototypes; raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise SkmError(
            f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C superkmeans_amd/csrc`"
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _PROTOTYPES.items():
        fn = getattr(lib, name)  # AttributeError here means header and library disagree
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        msg = load().skm_last_error()
        raise SkmError(f"libskm_hip error {rc}: {msg.decode() if msg else ''}")


class DeviceArray:
    """A typed device allocation owned by a Context."""

    def __init__(self, ctx, shape, dtype):
        self.ctx = ctx
        self.shape = tuple(int(s) for s in (shape if isinstance(shape, (tuple, list)) else (shape,)))
        self.dtype = np.dtype(dtype)
        self.nbytes = int(np.prod(self.shape, dtype=np.int64)) * self.dtype.itemsize
        p = c_void_p()
        check(ctx.lib.skm_malloc(ctx.handle, self.nbytes, ctypes.byref(p)))
        self.ptr = p.value
        ctx._live.append(self)

    @property
    def size(self):
        return int(np.prod(self.shape, dtype=np.int64))

    def upload(self, host):
        host = np.ascontiguousarray(host, dtype=self.dtype)
        if host.nbytes != self.nbytes:
            raise ValueError(f"upload size mismatch: {host.nbytes} != {self.nbytes}")
        check(self.ctx.lib.skm_upload(self.ctx.handle, self.ptr, host.ctypes.data, self.nbytes))
        return self

    def download(self, count=None):
        shape = self.shape if count is None else (int(count),) + self.shape[1:]
        out = np.empty(shape, dtype=self.dtype)
        check(self.ctx.lib.skm_download(self.ctx.handle, out.ctypes.data, self.ptr, out.nbytes))
        return out

    def offset(self, elements):
        """Device address `elements` items past the start."""
        return self.ptr + int(elements) * self.dtype.itemsize

    def free(self):
        if self.ptr:
            check(self.ctx.lib.skm_free(self.ctx.handle, self.ptr))
            self.ptr = None
            try:
                self.ctx._live.remove(self)
            except ValueError:
                pass


class Context:
    """One device + stream + workspace (skm_ctx)."""

    def __init__(self, device=0):
        self.lib = load()
        h = c_void_p()
        check(self.lib.skm_ctx_create(device, ctypes.byref(h)))
        self.handle = h.value
        self._live = []

    def close(self):
        if self.handle:
            for a in list(self._live):
                a.free()
            check(self.lib.skm_ctx_destroy(self.handle))
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def empty(self, shape, dtype=np.float32):
        return DeviceArray(self, shape, dtype)

    def array(self, host, dtype=None):
        host = np.ascontiguousarray(host, dtype=dtype if dtype is not None else host.dtype)
        return DeviceArray(self, host.shape, host.dtype).upload(host)

    def sync(self):
        check(self.lib.skm_sync(self.handle))

    def prof_enable(self, on=True):
        check(self.lib.skm_prof_enable(self.handle, 1 if on else 0))

    def prof_reset(self):
        check(self.lib.skm_prof_reset(self.handle))

    def prof(self):
        """Returns {scope: (milliseconds, calls)} of the device timers."""
        need = c_size_t()
        check(self.lib.skm_prof_dump(self.handle, None, 0, ctypes.byref(need)))
        buf = ctypes.create_string_buffer(need.value + 1)
        check(self.lib.skm_prof_dump(self.handle, buf, len(buf), ctypes.byref(need)))
        out = {}
        for item in buf.value.decode().split(";"):
            if not item:
                continue
            name, rest = item.split("=")
            ms, calls = rest.split("/")
            out[name] = (float(ms), int(calls))
        return out


def device_count():
    n = c_int()
    rc = load().skm_device_count(ctypes.byref(n))
    return n.value if rc == 0 else 0
