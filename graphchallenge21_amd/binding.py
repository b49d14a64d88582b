"""ctypes binding of include/spdnn.h."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))

KERNEL_AUTO, KERNEL_GATHER, KERNEL_BAND, KERNEL_BLOCK, KERNEL_TILED = 0, 1, 2, 3, 4

_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(dtype=np.uint8, flags="C_CONTIGUOUS")


class SpdnnError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("spdnn error %d: %s" % (code, message))
        self.code = code
        self.message = message


class LayerPlan(C.Structure):
    _fields_ = [("kernel", C.c_int32), ("max_row_nnz", C.c_int32), ("regular", C.c_int32),
                ("uniform_value", C.c_int32), ("value", C.c_float), ("exact_products", C.c_int32),
                ("band_halo", C.c_int32), ("nnz", C.c_int64), ("plan_bytes", C.c_int64),
                ("block_form", C.c_int32), ("fuse_next", C.c_int32), ("common_order", C.c_int32)]


class RunOptions(C.Structure):
    _fields_ = [("prune", C.c_int32), ("first_layer", C.c_int32), ("n_layers", C.c_int32),
                ("collect_counts", C.c_int32), ("time_layers", C.c_int32),
                ("compact_threshold", C.c_float), ("fuse_layers", C.c_int32), ("persist_wait_us", C.c_int32),
                ("reserved", C.c_int32 * 2)]


class RunResult(C.Structure):
    _fields_ = [("layers_run", C.c_int32), ("compactions", C.c_int32), ("active_rows", C.c_int64),
                ("carried_rows", C.c_int64), ("ms_total", C.c_float), ("ms_kernels", C.c_float),
                ("alg_bytes", C.c_double), ("edges", C.c_double), ("launches", C.c_int32), ("fused_pairs", C.c_int32),
                ("persistent_launches", C.c_int32), ("persistent_fallbacks", C.c_int32),
                ("resident_launches", C.c_int32), ("reserved", C.c_int32)]


def lib_path():
    return os.path.join(_HERE, "libspdnn.so")


_lib = None


def load_library():
    """Loads the in-tree libspdnn.so; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise SpdnnError(-1, "libspdnn.so is not built: run graphchallenge21_amd.build() "
                             "(or `make -C graphchallenge21_amd/csrc`)")
    lib = C.CDLL(path)
    vp = C.c_void_p
    lib.spdnn_last_error.restype = C.c_char_p
    sig = {
        "spdnn_version": ([], C.c_int),
        "spdnn_create": ([C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, C.POINTER(vp)], C.c_int),
        "spdnn_destroy": ([vp], C.c_int),
        "spdnn_reference_bias": ([C.c_int, C.POINTER(C.c_float)], C.c_int),
        "spdnn_set_layer_csr": ([vp, C.c_int, _i32p, _i32p, _f32p], C.c_int),
        "spdnn_load_layer_tsv": ([vp, C.c_int, C.c_char_p], C.c_int),
        "spdnn_load_layers_bin": ([vp, C.c_char_p, C.c_int, C.c_int, C.c_int64], C.c_int),
        "spdnn_weight_file_name": ([C.c_char_p, C.c_int, C.c_int, C.c_char_p, C.c_int], C.c_int),
        "spdnn_synth_layers": ([vp, C.c_uint64, C.c_int, C.c_int, C.c_int, C.c_float], C.c_int),
        "spdnn_synth_layer_csr": ([C.c_uint64, C.c_int, C.c_int, C.c_int, C.c_float, _i32p, _i32p, _f32p], C.c_int),
        "spdnn_inspect": ([vp], C.c_int),
        "spdnn_set_force_kernel": ([vp, C.c_int], C.c_int),
        "spdnn_load_layers_tsv": ([vp, C.c_char_p, C.c_int, C.c_int], C.c_int),
        "spdnn_read_features_tsv": ([C.c_char_p, C.c_int, C.c_int, _f32p, C.POINTER(C.c_int64)], C.c_int),
        "spdnn_set_plan_window": ([vp, C.c_int], C.c_int),
        "spdnn_get_plan_memory": ([vp, C.POINTER(C.c_int), C.POINTER(C.c_int64), C.POINTER(C.c_int64)], C.c_int),
        "spdnn_get_layer_plan": ([vp, C.c_int, C.POINTER(LayerPlan)], C.c_int),
        "spdnn_get_band_plan": ([vp, C.c_int, _i32p, _i32p, _u8p], C.c_int),
        "spdnn_get_band_pairs": ([vp, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int),
                                 C.POINTER(C.c_int), C.c_void_p, C.c_void_p], C.c_int),
        "spdnn_get_band_quads": ([vp, C.c_int, C.POINTER(C.c_int), C.c_void_p, C.c_void_p], C.c_int),
        "spdnn_get_layer_dst": ([vp, C.c_int, _i32p], C.c_int),
        "spdnn_get_layer_slots": ([vp, C.c_int, C.POINTER(C.c_int)], C.c_int),
        "spdnn_get_input_labelling": ([vp, C.c_int, _i32p], C.c_int),
        "spdnn_hash_reorder": ([C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int)], C.c_int),
        "spdnn_set_features_dense": ([vp, _f32p, C.c_int], C.c_int),
        "spdnn_load_features_tsv": ([vp, C.c_char_p, C.c_int], C.c_int),
        "spdnn_load_features_bin": ([vp, C.c_char_p, C.c_int], C.c_int),
        "spdnn_synth_features": ([vp, C.c_uint64, C.c_int, C.c_float, C.c_float], C.c_int),
        "spdnn_synth_features_host": ([C.c_uint64, C.c_int, C.c_int64, C.c_int64, C.c_float, C.c_float, _f32p], C.c_int),
        "spdnn_default_run_options": ([C.POINTER(RunOptions)], C.c_int),
        "spdnn_run": ([vp, C.POINTER(RunOptions), C.POINTER(RunResult)], C.c_int),
        "spdnn_get_active_count": ([vp, C.c_int, C.POINTER(C.c_int64)], C.c_int),
        "spdnn_get_categories": ([vp, C.c_void_p, C.c_int64, C.POINTER(C.c_int64)], C.c_int),
        "spdnn_get_activations": ([vp, _i32p, C.c_int, _f32p], C.c_int),
        "spdnn_get_activations_noalloc": ([vp, _i32p, C.c_int, _f32p], C.c_int),
        "spdnn_get_layer_times": ([vp, _f32p, C.c_int], C.c_int),
        "spdnn_get_band_tuning": ([vp, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)], C.c_int),
        "spdnn_write_categories": ([vp, C.c_char_p], C.c_int),
        "spdnn_receptive_field": ([vp, C.c_int, C.c_int, _i32p, C.c_int, _i32p, C.c_int64, C.POINTER(C.c_int64)], C.c_int),
        "spdnn_measure_copy_bandwidth": ([C.c_int64, C.c_int, C.POINTER(C.c_double)], C.c_int),
        "spdnn_measure_buffer_copy_bandwidth": ([vp, C.c_int, C.POINTER(C.c_double)], C.c_int),
        "spdnn_device_info": ([C.c_char_p, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int64)], C.c_int),
        "spdnn_get_feature_placement": ([vp, C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int64)], C.c_int),
        "spdnn_device_alloc_calls": ([C.POINTER(C.c_int64)], C.c_int),
        "spdnn_device_memory": ([C.POINTER(C.c_int64), C.POINTER(C.c_int64)], C.c_int),
        "spdnn_device_synchronize": ([], C.c_int),
    }
    for name, (args, res) in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = res
    _lib = lib
    return lib


def _check(rc):
    if rc != 0:
        raise SpdnnError(rc, load_library().spdnn_last_error().decode(errors="replace"))


def reference_bias(neuron):
    b = C.c_float()
    _check(load_library().spdnn_reference_bias(neuron, C.byref(b)))
    return b.value


def hash_reorder(v, buckets, domain):
    out = C.c_int()
    _check(load_library().spdnn_hash_reorder(v, buckets, domain, C.byref(out)))
    return out.value


def weight_file_name(data_dir, neuron, layer):
    buf = C.create_string_buffer(4096)
    _check(load_library().spdnn_weight_file_name(data_dir.encode(), neuron, layer, buf, 4096))
    return buf.value.decode()


def synth_layer_csr(seed, layer, neuron, nnz_per_row=32, value=0.0625):
    rowptr = np.empty(neuron + 1, np.int32)
    col = np.empty(neuron * nnz_per_row, np.int32)
    val = np.empty(neuron * nnz_per_row, np.float32)
    _check(load_library().spdnn_synth_layer_csr(seed, layer, neuron, nnz_per_row, value, rowptr, col, val))
    return rowptr, col, val


def synth_features_host(seed, neuron, row_begin, nrows, dmin=0.10, dmax=0.25):
    out = np.empty((nrows, neuron), np.float32)
    _check(load_library().spdnn_synth_features_host(seed, neuron, row_begin, nrows, dmin, dmax, out))
    return out


def read_features_tsv(path, neuron, batch):
    """(dense batch x neuron fp32, lines stored) of a feature file in the challenge format."""
    out = np.empty((batch, neuron), np.float32)
    kept = C.c_int64()
    _check(load_library().spdnn_read_features_tsv(str(path).encode(), neuron, batch, out, C.byref(kept)))
    return out, kept.value


def measure_copy_bandwidth(nbytes=1 << 30, reps=10):
    g = C.c_double()
    _check(load_library().spdnn_measure_copy_bandwidth(nbytes, reps, C.byref(g)))
    return g.value


def device_info():
    name = C.create_string_buffer(256)
    cu, mem = C.c_int(), C.c_int64()
    _check(load_library().spdnn_device_info(name, 256, C.byref(cu), C.byref(mem)))
    return name.value.decode(), cu.value, mem.value


def device_alloc_calls():
    """Device allocations the library has made in this process so far."""
    c = C.c_int64()
    _check(load_library().spdnn_device_alloc_calls(C.byref(c)))
    return c.value


def device_memory():
    """(free, total) device memory in bytes."""
    free, total = C.c_int64(), C.c_int64()
    _check(load_library().spdnn_device_memory(C.byref(free), C.byref(total)))
    return free.value, total.value


class Network:
    """One network handle: create -> set layers -> inspect -> set features -> run -> read back."""

    def __init__(self, neuron, max_batch, layers, bias=None, clamp=32.0, force_kernel=KERNEL_AUTO):
        self._lib = load_library()
        self.neuron, self.max_batch, self.layers = neuron, max_batch, layers
        self.bias = reference_bias(neuron) if bias is None else float(bias)
        h = C.c_void_p()
        _check(self._lib.spdnn_create(neuron, max_batch, layers, self.bias, clamp, C.byref(h)))
        self._h = h
        self.batch = 0
        if force_kernel != KERNEL_AUTO:
            _check(self._lib.spdnn_set_force_kernel(self._h, force_kernel))

    def close(self):
        if getattr(self, "_h", None):
            self._lib.spdnn_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    # weights
    def set_layer_csr(self, layer, rowptr, col, val):
        _check(self._lib.spdnn_set_layer_csr(
            self._h, layer, np.ascontiguousarray(rowptr, np.int32),
            np.ascontiguousarray(col, np.int32) if len(col) else np.zeros(1, np.int32),
            np.ascontiguousarray(val, np.float32) if len(val) else np.zeros(1, np.float32)))

    def load_layer_tsv(self, layer, path):
        _check(self._lib.spdnn_load_layer_tsv(self._h, layer, path.encode()))

    def load_layers_tsv(self, data_dir, first=0, count=None):
        """Layers [first, first+count) from <data_dir>/neuron<N>/n<N>-l<l+1>.tsv, parsed in parallel."""
        count = self.layers - first if count is None else count
        _check(self._lib.spdnn_load_layers_tsv(self._h, str(data_dir).encode(), first, count))

    def load_layers_bin(self, path, first=0, count=None, nnz_per_layer=0):
        count = self.layers - first if count is None else count
        _check(self._lib.spdnn_load_layers_bin(self._h, path.encode(), first, count, nnz_per_layer))

    def synth_layers(self, seed, first=0, count=None, nnz_per_row=32, value=0.0625):
        count = self.layers - first if count is None else count
        _check(self._lib.spdnn_synth_layers(self._h, seed, first, count, nnz_per_row, value))

    def inspect(self):
        _check(self._lib.spdnn_inspect(self._h))

    def layer_plan(self, layer):
        p = LayerPlan()
        _check(self._lib.spdnn_get_layer_plan(self._h, layer, C.byref(p)))
        return p

    def band_plan(self, layer):
        k = self.layer_plan(layer).max_row_nnz
        in_pos = np.empty(self.neuron, np.int32)
        out_at = np.empty(self.neuron, np.int32)
        sel = np.empty(self.neuron * k, np.uint8)
        _check(self._lib.spdnn_get_band_plan(self._h, layer, in_pos, out_at, sel))
        return in_pos, out_at, sel.reshape(self.neuron, k)

    def band_pairs(self, layer):
        """(steps, records uint32[neuron/2][stride], weights float32[neuron/2][padded_steps][2] or None)."""
        steps, stride, padded, has_w = C.c_int(), C.c_int(), C.c_int(), C.c_int()
        _check(self._lib.spdnn_get_band_pairs(self._h, layer, C.byref(steps), C.byref(stride), C.byref(padded),
                                              C.byref(has_w), None, None))
        rec = np.empty((self.neuron // 2, stride.value), np.uint32)
        w = np.empty((self.neuron // 2, padded.value, 2), np.float32) if has_w.value else None
        _check(self._lib.spdnn_get_band_pairs(self._h, layer, None, None, None, None, rec.ctypes.data,
                                              None if w is None else w.ctypes.data))
        return steps.value, rec, w

    def band_quads(self, layer):
        """(groups, columns uint32[neuron/4][groups][4] as byte offsets (column * 64), weights
        float32[neuron/4][groups][4 steps][4 outputs]); groups = 0: the layer has no QUAD form."""
        groups = C.c_int()
        _check(self._lib.spdnn_get_band_quads(self._h, layer, C.byref(groups), None, None))
        g = groups.value
        cols = np.empty((self.neuron // 4, g, 4), np.uint32)
        w = np.empty((self.neuron // 4, g, 4, 4), np.float32)
        if g:
            _check(self._lib.spdnn_get_band_quads(self._h, layer, None, cols.ctypes.data, w.ctypes.data))
        return g, cols, w

    def receptive_field(self, first_layer, n_layers, out_neurons):
        """Input neurons of layer first_layer that the given output neurons of layer
        first_layer + n_layers - 1 depend on (ascending)."""
        outs = np.ascontiguousarray(out_neurons, dtype=np.int32)
        res = np.empty(self.neuron, np.int32)
        cnt = C.c_int64()
        _check(self._lib.spdnn_receptive_field(self._h, first_layer, n_layers, outs, len(outs), res, len(res), C.byref(cnt)))
        return res[:cnt.value].copy()

    def feature_placement(self):
        """(paired, candidates, search_peak_bytes): whether the buffer halves lie in different memory regions,
        how many half-buffers the search allocated and how much device memory it held at its peak."""
        paired, cand, peak = C.c_int(), C.c_int(), C.c_int64()
        _check(self._lib.spdnn_get_feature_placement(self._h, C.byref(paired), C.byref(cand), C.byref(peak)))
        return bool(paired.value), cand.value, peak.value

    def set_plan_window(self, slots):
        """0 = every plan resident; 2..64 = that many device slots, plans streamed from pinned memory."""
        _check(self._lib.spdnn_set_plan_window(self._h, int(slots)))

    def plan_memory(self):
        """(window, device_bytes, pinned_bytes) of the uploaded plans."""
        w, d, h = C.c_int(), C.c_int64(), C.c_int64()
        _check(self._lib.spdnn_get_plan_memory(self._h, C.byref(w), C.byref(d), C.byref(h)))
        return w.value, d.value, h.value

    def layer_dst(self, layer):
        p = self.layer_plan(layer)
        slots = self.neuron
        if p.kernel in (KERNEL_BLOCK, KERNEL_TILED):
            slots = C.c_int()
            _check(self._lib.spdnn_get_layer_slots(self._h, layer, C.byref(slots)))
            slots = slots.value
        dst = np.empty(slots, np.int32)
        _check(self._lib.spdnn_get_layer_dst(self._h, layer, dst))
        return dst

    def input_labelling(self, layer):
        p = np.empty(self.neuron, np.int32)
        _check(self._lib.spdnn_get_input_labelling(self._h, layer, p))
        return p

    # features
    def set_features_dense(self, features):
        f = np.ascontiguousarray(features, np.float32)
        if f.ndim != 2 or f.shape[1] != self.neuron:
            raise ValueError("features must be batch x neuron")
        _check(self._lib.spdnn_set_features_dense(self._h, f, f.shape[0]))
        self.batch = f.shape[0]

    def load_features_tsv(self, path, batch):
        _check(self._lib.spdnn_load_features_tsv(self._h, path.encode(), batch))
        self.batch = batch

    def load_features_bin(self, path, batch):
        _check(self._lib.spdnn_load_features_bin(self._h, path.encode(), batch))
        self.batch = batch

    def synth_features(self, seed, batch, dmin=0.10, dmax=0.25):
        _check(self._lib.spdnn_synth_features(self._h, seed, batch, dmin, dmax))
        self.batch = batch

    # inference
    def run(self, prune=True, first_layer=0, n_layers=-1, collect_counts=False, time_layers=False,
            compact_threshold=0.75, fuse_layers=0, persist_wait_us=0):
        opt = RunOptions()
        _check(self._lib.spdnn_default_run_options(C.byref(opt)))
        opt.prune, opt.first_layer, opt.n_layers = int(prune), first_layer, n_layers
        opt.collect_counts, opt.time_layers = int(collect_counts), int(time_layers)
        opt.compact_threshold = compact_threshold
        opt.fuse_layers = fuse_layers
        opt.persist_wait_us = persist_wait_us
        res = RunResult()
        _check(self._lib.spdnn_run(self._h, C.byref(opt), C.byref(res)))
        return res

    def active_count(self, layer):
        c = C.c_int64()
        _check(self._lib.spdnn_get_active_count(self._h, layer, C.byref(c)))
        return c.value

    def categories(self):
        n = C.c_int64()
        _check(self._lib.spdnn_get_categories(self._h, None, 0, C.byref(n)))
        ids = np.empty(max(n.value, 1), np.int32)
        _check(self._lib.spdnn_get_categories(self._h, ids.ctypes.data_as(C.c_void_p), ids.size, C.byref(n)))
        return ids[:n.value].copy()

    def activations(self, rows):
        rows = np.ascontiguousarray(rows, np.int32)
        out = np.empty((len(rows), self.neuron), np.float32)
        if len(rows):
            _check(self._lib.spdnn_get_activations(self._h, rows, len(rows), out))
        return out

    def activations_noalloc(self, rows):
        """spdnn_get_activations_noalloc: the same rows through the library's static scratch memory."""
        rows = np.ascontiguousarray(rows, np.int32)
        out = np.empty((len(rows), self.neuron), np.float32)
        if len(rows):
            _check(self._lib.spdnn_get_activations_noalloc(self._h, rows, len(rows), out))
        return out

    def buffer_copy_bandwidth(self, reps=3):
        """GB/s (read + written) of a plain copy of one work buffer into the other."""
        g = C.c_double()
        _check(self._lib.spdnn_measure_buffer_copy_bandwidth(self._h, reps, C.byref(g)))
        return g.value

    def layer_times(self):
        ms = np.empty(self.layers, np.float32)
        _check(self._lib.spdnn_get_layer_times(self._h, ms, self.layers))
        return ms

    def band_tuning(self):
        """[(row_blocks, shape, seglen), ...] measured so far."""
        out, i = [], 0
        while True:
            a, b, c = C.c_int(), C.c_int(), C.c_int()
            if self._lib.spdnn_get_band_tuning(self._h, i, C.byref(a), C.byref(b), C.byref(c)) != 0:
                return out
            out.append((a.value, b.value, c.value))
            i += 1

    def write_categories(self, path):
        _check(self._lib.spdnn_write_categories(self._h, path.encode()))
