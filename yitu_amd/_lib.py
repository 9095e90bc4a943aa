"""ctypes binding of libyitu_hip.so and the small amount of torch plumbing
(device pointers, current stream, cached workspace) shared by the op modules.

There is no CPU fallback: if the library is missing or a tensor is not on a HIP
device the call raises.
"""
import ctypes
import os
import threading
import weakref

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libyitu_hip.so")
_lib = None
_lock = threading.Lock()
# The C ABI these bindings were written for (yitu_abi_version() of include/yitu_hip.h). A
# library of another version has other argument lists: calling it would hand the kernels
# shifted pointers, so it is refused at load time.
ABI_VERSION = 4

c_i64 = ctypes.c_int64
c_int = ctypes.c_int
c_f32 = ctypes.c_float
c_size = ctypes.c_size_t
c_ptr = ctypes.c_void_p


def lib():
    """Loads the HIP library; raises if it has not been built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise RuntimeError(
                        "libyitu_hip.so is not built; run `python -m yitu_amd.build` "
                        "(there is no CPU fallback)")
                l = ctypes.CDLL(LIB_PATH)
                l.yitu_abi_version.restype = ctypes.c_int
                found = l.yitu_abi_version()
                if found != ABI_VERSION:
                    raise RuntimeError(
                        "libyitu_hip.so has ABI version %d, these bindings need %d; rebuild it "
                        "with `python -m yitu_amd.build --force`" % (found, ABI_VERSION))
                l.yitu_last_error.restype = ctypes.c_char_p
                _lib = l
    return _lib


def _declare(name, restype=ctypes.c_int):
    fn = getattr(lib(), name)
    fn.restype = restype
    return fn


def check(rc, what):
    if rc != 0:
        msg = lib().yitu_last_error().decode("utf-8", "replace")
        raise RuntimeError("%s failed (code %d): %s" % (what, rc, msg))


def ptr(t):
    """Device address of a tensor (None -> NULL)."""
    if t is None:
        return c_ptr(0)
    return c_ptr(t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device):
    """The current HIP stream of ``device`` as a pointer argument."""
    if _raw_stream is not None and device.index is not None:
        return c_ptr(_raw_stream(device.index))  # no Stream object on the way
    return c_ptr(torch.cuda.current_stream(device).cuda_stream)


def require_device(*tensors):
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise RuntimeError("expected a tensor on the GPU (HIP device), got %s" % t.device)
        if not t.is_contiguous():
            raise RuntimeError("expected a contiguous tensor")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError("tensors live on different devices: %s vs %s" % (dev, t.device))
    return dev


def require_dtype(t, dtype, name):
    if t.dtype != dtype:
        raise RuntimeError("%s must be %s, got %s" % (name, dtype, t.dtype))


def workspace(n_bytes, device):
    """Scratch buffer for one call; the caching allocator makes this cheap and
    stream-ordered reuse keeps concurrent ops on one stream from colliding."""
    n = max(int(n_bytes), 256)
    return torch.empty(n, dtype=torch.uint8, device=device)


# ---- state derived from a graph ----------------------------------------------------
# The widest row, the row plan, the by-source view and by-source weight copies are
# functions of the index tensors and are kept per tensor OBJECT (id, address, version
# counter) for as long as the tensor lives. The version counter moves when torch writes
# the tensor; it does NOT move when a buffer is refilled through its raw pointer, which is
# how every kernel of this library (yitu_coo_to_csr, the device sampler, ...), DLPack
# consumers and foreign extensions write. Whoever refills an index or weight tensor in
# place must call ``forget`` on it (graph_ext.forget also drops the by-source state);
# the builders in data/csr.py and the samplers return fresh tensors and need not.
#
# Derived buffers are built on the stream that was current at the time; a later use on
# another stream waits for the build through an event recorded right behind it.


class _Built:
    __slots__ = ("value", "event", "raw_stream")

    def __init__(self, value, device):
        self.value = value
        self.raw_stream = stream_ptr(device).value
        self.event = torch.cuda.Event()
        self.event.record(torch.cuda.current_stream(device))

    def get(self, device):
        if stream_ptr(device).value != self.raw_stream:  # two integers in the common case
            torch.cuda.current_stream(device).wait_event(self.event)
        return self.value


def forget(*tensors):
    """Drops every cached widest row and row plan derived from the given index tensors
    (call after refilling one of them in place through a raw pointer)."""
    idents = {id(t) for t in tensors if t is not None}
    for key in [k for k in _max_degree if k[0] in idents]:
        _max_degree.pop(key, None)
    for key in [k for k in _plans if k[0] in idents or k[3] in idents]:
        _plans.pop(key, None)


# Widest-row cache: the kernels skip their hub-row machinery when they are told
# that no row reaches the hub threshold. Computed once per indptr tensor.
_max_degree = {}


def max_degree(indptr):
    """Longest row of a CSR, computed once per ``indptr`` tensor. The entry lives as long
    as the tensor object: an address alone is no identity, the allocator hands a freed
    block to the next graph of the same size."""
    key = (id(indptr), indptr.data_ptr(), indptr.numel(), indptr._version)
    v = _max_degree.get(key)
    if v is None:
        if indptr.numel() <= 1:
            v = 0
        else:
            v = int((indptr[1:] - indptr[:-1]).max().item())
        _max_degree[key] = v
        weakref.finalize(indptr, _max_degree.pop, key, None)
    return v


# Row plans (band-ordered items of the long rows) are a function of the graph
# only: built on the device on first use and kept while the index tensor lives.
_plans = {}


def row_plan(indptr, indices, n_src, col_mask):
    """Device buffer holding the row plan of (indptr, indices), or None when no
    row reaches the planning threshold and the graph is small. A large graph without
    long rows still gets one: its header tells the row kernels whether most sources of
    a row lie near the row's own id, which decides how rows are dealt to the XCDs."""
    if max_degree(indptr) < 64 and indices.numel() < (1 << 20):
        return None
    key = (id(indices), indices.data_ptr(), indices._version, id(indptr), indptr.data_ptr(),
           indptr._version, int(n_src), int(col_mask))
    hit = _plans.get(key)
    if hit is not None:
        return hit.get(indices.device)
    L = lib()
    L.yitu_plan_bytes.restype = c_size
    L.yitu_plan_workspace_bytes.restype = c_size
    dev = indices.device
    nnz = indices.numel()
    plan = torch.empty(int(L.yitu_plan_bytes(c_i64(nnz))), dtype=torch.uint8, device=dev)
    ws = workspace(L.yitu_plan_workspace_bytes(c_i64(nnz)), dev)
    with torch.cuda.device(dev):
        rc = L.yitu_plan_build(ptr(plan), c_size(plan.numel()), ptr(indptr), ptr(indices),
                               c_i64(indptr.numel() - 1), c_i64(n_src), c_i64(nnz), c_int(col_mask),
                               ptr(ws), c_size(ws.numel()), stream_ptr(dev))
    check(rc, "yitu_plan_build")
    _plans[key] = _Built(plan, dev)
    weakref.finalize(indices, _plans.pop, key, None)
    return plan


def size_fn(name):
    fn = getattr(lib(), name)
    fn.restype = c_size
    return fn
