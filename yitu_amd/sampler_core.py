"""Drop-in for the reference's ``sampler_core`` extension module
(YiTu_GNN/YiTu_T/sampler_core.cpp:374-402): ``ParallelSampler`` with
``sample / reset / get_ret`` and ``TemporalGraphBlock`` accessors returning numpy
arrays, in every mode of the reference's constructor: most recent or uniformly drawn
neighbours (``recent``), cursors or binary search in later layers (``prop_time``),
snapshots of a sliding window (``num_history``, ``window_duration``). The uniform draws
are the reference's own (its per-thread ``rand_r`` streams are a function of
``num_thread_per_worker * num_workers``). ``GpuParallelSampler`` is the most-recent mode
with the T-CSR and the cursors on the device.
"""
import ctypes

import numpy as np

from . import _host


class TemporalGraphBlock:
    """COO block: ``row`` = root slot, ``col`` = index into ``nodes`` (roots first),
    ``eid``, ``ts``, ``dts`` (= root time - edge time, 0 for the roots), ``nodes``."""

    def __init__(self, row, col, eid, ts, dts, nodes, dim_in, dim_out):
        self._row, self._col, self._eid = row, col, eid
        self._ts, self._dts, self._nodes = ts, dts, nodes
        self._dim_in, self._dim_out = int(dim_in), int(dim_out)

    def row(self):
        return self._row.copy()

    def col(self):
        return self._col.copy()

    def eid(self):
        return self._eid.copy()

    def ts(self):
        return self._ts.copy()

    def dts(self):
        return self._dts.copy()

    def nodes(self):
        return self._nodes.copy()

    def dim_in(self):
        return self._dim_in

    def dim_out(self):
        return self._dim_out

    # phase timers of the reference block; not collected here
    def tot_time(self):
        return 0.0

    ptr_time = search_time = sample_time = coo_time = tot_time


class ParallelSampler:
    def __init__(self, indptr, indices, eid, ts, num_thread_per_worker, num_workers, num_layers,
                 num_neighbors, recent, prop_time, num_history, window_duration):
        if int(num_history) < 1:
            raise ValueError("num_history must be at least 1")
        self._indptr = np.ascontiguousarray(indptr, dtype=np.int32)
        self._indices = np.ascontiguousarray(indices, dtype=np.int32)
        self._eid = np.ascontiguousarray(eid, dtype=np.int32)
        self._ts = np.ascontiguousarray(ts, dtype=np.float32)
        fan = np.ascontiguousarray(num_neighbors, dtype=np.int32)
        if fan.shape[0] < num_layers:
            raise ValueError("num_neighbors needs one entry per layer")
        p = lambda a: ctypes.c_void_p(a.ctypes.data)
        create = _host.lib().yitu_sampler_create_modes
        create.restype = ctypes.c_void_p
        self._h = create(
            p(self._indptr), p(self._indices), p(self._eid), p(self._ts),
            ctypes.c_int64(self._indptr.shape[0] - 1), ctypes.c_int64(self._indices.shape[0]),
            ctypes.c_int(int(num_thread_per_worker) * int(num_workers)), ctypes.c_int(num_layers),
            p(fan), ctypes.c_int(int(bool(recent))), ctypes.c_int(int(bool(prop_time))),
            ctypes.c_int(int(num_history)), ctypes.c_float(float(window_duration)))
        if not self._h:
            raise RuntimeError("invalid T-CSR passed to ParallelSampler")
        self._ret = []

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            _host.lib().yitu_sampler_destroy(ctypes.c_void_p(h))
            self._h = None

    def reset(self):
        _host.lib().yitu_sampler_reset(ctypes.c_void_p(self._h))

    def sample(self, root_nodes, root_ts):
        nodes = np.ascontiguousarray(root_nodes, dtype=np.int32)
        ts = np.ascontiguousarray(root_ts, dtype=np.float32)
        if nodes.shape != ts.shape or nodes.ndim != 1:
            raise ValueError("root_nodes and root_ts must be 1-D and equally long")
        L = _host.lib()
        rc = L.yitu_sampler_sample(ctypes.c_void_p(self._h), ctypes.c_void_p(nodes.ctypes.data),
                                   ctypes.c_void_p(ts.ctypes.data), ctypes.c_int64(nodes.shape[0]))
        if rc != 0:
            raise RuntimeError("sample failed: %s" %
                               L.yitu_sampler_last_error(ctypes.c_void_p(self._h)).decode())
        self._ret = []
        for b in range(L.yitu_sampler_num_blocks(ctypes.c_void_p(self._h))):
            ne, din, dout = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
            L.yitu_sampler_block_sizes(ctypes.c_void_p(self._h), b, ctypes.byref(ne),
                                       ctypes.byref(din), ctypes.byref(dout))
            row = np.empty(ne.value, np.int32)
            col = np.empty(ne.value, np.int32)
            eid = np.empty(ne.value, np.int32)
            bts = np.empty(din.value, np.float32)
            dts = np.empty(din.value, np.float32)
            bn = np.empty(din.value, np.int32)
            p = lambda a: ctypes.c_void_p(a.ctypes.data)
            L.yitu_sampler_block_copy(ctypes.c_void_p(self._h), b, p(row), p(col), p(eid), p(bts),
                                      p(dts), p(bn))
            self._ret.append(TemporalGraphBlock(row, col, eid, bts, dts, bn, din.value, dout.value))

    def get_ret(self):
        return list(self._ret)


class DeviceTemporalGraphBlock:
    """A sampled block whose arrays are torch tensors on the GPU; the accessors
    mirror TemporalGraphBlock (``.cpu_block()`` converts to the numpy form)."""

    def __init__(self, row, col, eid, ts, dts, nodes, dim_in, dim_out):
        self._a = (row, col, eid, ts, dts, nodes)
        self._dim_in, self._dim_out = int(dim_in), int(dim_out)

    def row(self):
        return self._a[0]

    def col(self):
        return self._a[1]

    def eid(self):
        return self._a[2]

    def ts(self):
        return self._a[3]

    def dts(self):
        return self._a[4]

    def nodes(self):
        return self._a[5]

    def dim_in(self):
        return self._dim_in

    def dim_out(self):
        return self._dim_out

    def cpu_block(self):
        return TemporalGraphBlock(*[t.cpu().numpy() for t in self._a], self._dim_in, self._dim_out)


class GpuParallelSampler:
    """ParallelSampler with the T-CSR and the cursors in device memory: same constructor
    arguments, same results bit for bit in every mode (the uniform draws included: a
    root's generator state is reached by skipping ahead in its nominal thread's
    sequence), blocks returned as DeviceTemporalGraphBlock. The most-recent,
    single-snapshot mode runs as one call per layer (yitu_tsample_recent); the other
    modes string yitu_tsample_advance / yitu_tsample_window together per layer and
    snapshot the way the reference's sample() does (sampler_core.cpp:337-359)."""

    def __init__(self, indptr, indices, eid, ts, num_thread_per_worker, num_workers, num_layers,
                 num_neighbors, recent, prop_time, num_history, window_duration, device="cuda"):
        import torch
        if int(num_history) < 1:
            raise ValueError("num_history must be at least 1")
        if len(num_neighbors) < num_layers:
            raise ValueError("num_neighbors needs one entry per layer")
        self._dev = torch.device(device)
        to = lambda a, dt: torch.as_tensor(np.ascontiguousarray(a, dtype=dt)).to(self._dev)
        self._indptr = to(indptr, np.int32)
        self._indices = to(indices, np.int32)
        self._eid = to(eid, np.int32)
        self._ts = to(ts, np.float32)
        self._n_nodes = self._indptr.numel() - 1
        self._fan = [int(x) for x in num_neighbors[:num_layers]]
        self._prop_time = bool(prop_time)
        self._recent = bool(recent)
        self._hist = int(num_history)
        self._window = float(np.float32(window_duration))
        self._threads = max(1, int(num_thread_per_worker) * int(num_workers))
        self._simple = self._recent and self._hist == 1 and abs(self._window) <= 1e-7
        # cursor k of a node, k = 0 .. num_history (ts_ptr of the reference, :57-58)
        self._cursors = torch.empty(self._hist + 1, max(self._n_nodes, 1), dtype=torch.int32,
                                    device=self._dev)
        self._cursor = self._cursors[self._hist]
        self._ret = []
        self.reset()

    def reset(self):
        from . import _lib
        for k in range(self._hist + 1):
            rc = _lib.lib().yitu_tsample_reset(_lib.ptr(self._cursors[k]), _lib.ptr(self._indptr),
                                               _lib.c_i64(self._n_nodes),
                                               _lib.stream_ptr(self._dev))
            _lib.check(rc, "yitu_tsample_reset")

    def _outputs(self, n, fan):
        import torch
        i32 = lambda m: torch.empty(max(m, 1), dtype=torch.int32, device=self._dev)
        f32 = lambda m: torch.empty(max(m, 1), dtype=torch.float32, device=self._dev)
        return (i32(n * fan), i32(n * fan), i32(n * fan), f32(n * (fan + 1)), f32(n * (fan + 1)),
                i32(n * (fan + 1)), torch.empty(1, dtype=torch.int64, device=self._dev))

    def _block(self, outs, n):
        row, col, eid, ts, dts, nodes, count = outs
        m = int(count.item())
        if m < 0:
            raise RuntimeError("sample failed: a root node id is out of range")
        return DeviceTemporalGraphBlock(row[:m], col[:m], eid[:m], ts[:n + m], dts[:n + m],
                                        nodes[:n + m], n + m, n)

    def _layer(self, roots, root_ts, fan):
        import torch
        from . import _lib
        n = roots.numel()
        outs = self._outputs(n, fan)
        ws = _lib.workspace(_lib.size_fn("yitu_tsample_workspace_bytes")(_lib.c_i64(n)), self._dev)
        with torch.cuda.device(self._dev):
            rc = _lib.lib().yitu_tsample_recent(
                *[_lib.ptr(t) for t in outs], _lib.ptr(self._cursor), _lib.ptr(self._indptr),
                _lib.ptr(self._indices), _lib.ptr(self._eid), _lib.ptr(self._ts),
                _lib.c_i64(self._n_nodes), _lib.ptr(roots), _lib.ptr(root_ts), _lib.c_i64(n),
                _lib.c_int(fan), _lib.c_int(int(self._prop_time)), _lib.ptr(ws),
                _lib.c_size(ws.numel()), _lib.stream_ptr(self._dev))
        _lib.check(rc, "yitu_tsample_recent")
        return self._block(outs, n)

    def _advance(self, k, roots, root_ts, offset):
        import torch
        from . import _lib
        with torch.cuda.device(self._dev):
            rc = _lib.lib().yitu_tsample_advance(
                _lib.ptr(self._cursors[k]), _lib.ptr(self._indptr), _lib.ptr(self._ts),
                _lib.c_i64(self._n_nodes), _lib.ptr(roots), _lib.ptr(root_ts),
                _lib.c_i64(roots.numel()), _lib.c_f32(offset), _lib.stream_ptr(self._dev))
        _lib.check(rc, "yitu_tsample_advance")

    def _snapshot(self, roots, root_ts, fan, use_ptr, i):
        import torch
        from . import _lib
        n = roots.numel()
        outs = self._outputs(n, fan)
        ws = _lib.workspace(_lib.size_fn("yitu_tsample_window_workspace_bytes")(_lib.c_i64(n)),
                            self._dev)
        offset = float(-np.float32(i) * np.float32(self._window))
        # the reference's static chunk of roots per thread, computed in float as it does (:239)
        chunk = int(np.ceil(np.float32(n) / np.float32(self._threads))) if n else 1
        lo = self._cursors[self._hist - 1 - i] if use_ptr else None
        hi = self._cursors[self._hist - i] if use_ptr else None
        with torch.cuda.device(self._dev):
            rc = _lib.lib().yitu_tsample_window(
                *[_lib.ptr(t) for t in outs], _lib.ptr(lo), _lib.ptr(hi), _lib.ptr(self._indptr),
                _lib.ptr(self._indices), _lib.ptr(self._eid), _lib.ptr(self._ts),
                _lib.c_i64(self._n_nodes), _lib.ptr(roots), _lib.ptr(root_ts), _lib.c_i64(n),
                _lib.c_int(fan), _lib.c_int(int(self._prop_time)), _lib.c_int(int(self._recent)),
                _lib.c_int(int(self._hist > 1)), _lib.c_f32(offset), _lib.c_f32(self._window),
                _lib.c_i64(chunk), _lib.ptr(ws), _lib.c_size(ws.numel()),
                _lib.stream_ptr(self._dev))
        _lib.check(rc, "yitu_tsample_window")
        return self._block(outs, n)

    def sample(self, root_nodes, root_ts):
        import torch
        roots = torch.as_tensor(root_nodes).to(self._dev, torch.int32).contiguous()
        ts = torch.as_tensor(root_ts).to(self._dev, torch.float32).contiguous()
        if roots.shape != ts.shape or roots.dim() != 1:
            raise ValueError("root_nodes and root_ts must be 1-D and equally long")
        self._ret = []
        if self._simple:
            for fan in self._fan:
                blk = self._layer(roots, ts, fan)
                self._ret.append(blk)
                # the next layer expands every node of this block (roots and neighbours)
                roots, ts = blk.nodes(), blk.ts()
            return
        H = self._hist
        first_layer = True
        for layer, fan in enumerate(self._fan):
            self._ret.extend([None] * H)
            n_blocks = len(self._ret)
            use_ptr = first_layer or (self._prop_time and H == 1) or self._recent
            first_layer = False

            def layer_roots(i):
                if layer == 0:
                    return roots, ts
                prev = self._ret[n_blocks - 1 - i - H]
                return prev.nodes(), prev.ts()

            if use_ptr:
                self._advance(H, *layer_roots(0), 0.0)
            for i in range(H):
                r, t = layer_roots(i)
                if use_ptr and abs(self._window) > 1e-7:
                    off = np.float32(-np.float32(i) * np.float32(self._window)) - np.float32(self._window)
                    self._advance(H - 1 - i, r, t, float(off))
                self._ret[n_blocks - 1 - i] = self._snapshot(r, t, fan, use_ptr, i)

    def get_ret(self):
        return list(self._ret)
