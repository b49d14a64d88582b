"""ctypes front end of the CPU oracle (oracle/spdnn_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
CPU-baseline leg of bench.py, never by the graphchallenge21_amd package.

Parity unpinned: read_weights_bin and read_features_bin follow the way the reference's library
benchmark reads its packed files, but no such file ships with the reference to check them against.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
REF_CHECK = os.path.join(_HERE, "_ref", "ref_check")

_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_u8p = np.ctypeslib.ndpointer(dtype=np.uint8, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")


def build(with_ref=True):
    """Compile liboracle.so (and oracle/_ref/ref_check when the reference is mounted)."""
    target = ["all"] if with_ref else ["liboracle.so"]
    subprocess.run(["make", "-s", "-C", _HERE] + target, check=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build(with_ref=False)
    lib = C.CDLL(_LIB_PATH)
    lib.orc_splitmix64.restype = C.c_uint64
    lib.orc_splitmix64.argtypes = [C.c_uint64]
    lib.orc_gen_layer_params.restype = None
    lib.orc_gen_layer_params.argtypes = [C.c_uint64, C.c_int, C.c_int, _i32p,
                                         C.POINTER(C.c_int), C.POINTER(C.c_int)]
    lib.orc_gen_layer_csr.restype = C.c_int
    lib.orc_gen_layer_csr.argtypes = [C.c_uint64, C.c_int, C.c_int, C.c_int, C.c_float, _i32p, _i32p, _f32p]
    lib.orc_gen_features.restype = None
    lib.orc_gen_features.argtypes = [C.c_uint64, C.c_int, C.c_int64, C.c_int64, C.c_float, C.c_float, _f32p]
    lib.orc_feature_threshold.restype = C.c_uint32
    lib.orc_feature_threshold.argtypes = [C.c_uint64, C.c_int64, C.c_float, C.c_float]
    lib.orc_hash_reorder.restype = C.c_int
    lib.orc_hash_reorder.argtypes = [C.c_int, C.c_int, C.c_int]
    lib.orc_count_tsv_triples.restype = C.c_int64
    lib.orc_count_tsv_triples.argtypes = [C.c_char_p]
    lib.orc_read_weight_tsv.restype = C.c_int64
    lib.orc_read_weight_tsv.argtypes = [C.c_char_p, C.c_int, C.c_int64, _i32p, _i32p, _f32p,
                                        C.POINTER(C.c_int), C.POINTER(C.c_int)]
    lib.orc_coo_to_csr.restype = C.c_int
    lib.orc_coo_to_csr.argtypes = [C.c_int64, C.c_int, _i32p, _i32p, _f32p, _i32p, _i32p, _f32p]
    lib.orc_read_features_tsv.restype = C.c_int64
    lib.orc_read_features_tsv.argtypes = [C.c_char_p, C.c_int, C.c_int, _f32p]
    lib.orc_relu_clamp.restype = C.c_float
    lib.orc_relu_clamp.argtypes = [C.c_float]
    lib.orc_set_threads.restype = None
    lib.orc_set_threads.argtypes = [C.c_int]
    lib.orc_get_threads.restype = C.c_int
    lib.orc_layer.restype = None
    lib.orc_layer.argtypes = [_f32p, C.c_int64, C.c_int, _i32p, _i32p, _f32p, C.c_float, _f32p, _i32p]
    lib.orc_compact.restype = C.c_int64
    lib.orc_compact.argtypes = [_f32p, C.c_int64, C.c_int, _i32p, _i32p, _f32p, _i32p]
    lib.orc_need_access.restype = None
    lib.orc_need_access.argtypes = [C.c_int, _i32p, _i32p, _u8p, _u8p]
    return lib


_lib = _load()


def set_threads(n):
    _lib.orc_set_threads(int(n))


def get_threads():
    return int(_lib.orc_get_threads())


def splitmix64(x):
    return int(_lib.orc_splitmix64(C.c_uint64(x & 0xFFFFFFFFFFFFFFFF)))


def gen_layer_params(seed, layer, neuron):
    perm = np.empty(neuron, dtype=np.int32)
    o, s = C.c_int(), C.c_int()
    _lib.orc_gen_layer_params(seed, layer, neuron, perm, C.byref(o), C.byref(s))
    return perm, o.value, s.value


def gen_layer_csr(seed, layer, neuron, nnz_per_row=32, value=0.0625):
    """CSR (row = output neuron, col = input neuron ascending) of synthetic layer `layer`."""
    rowptr = np.empty(neuron + 1, dtype=np.int32)
    col = np.empty(neuron * nnz_per_row, dtype=np.int32)
    val = np.empty(neuron * nnz_per_row, dtype=np.float32)
    rc = _lib.orc_gen_layer_csr(seed, layer, neuron, nnz_per_row, value, rowptr, col, val)
    if rc != 0:
        raise ValueError("orc_gen_layer_csr failed: %d" % rc)
    return rowptr, col, val


def gen_features(seed, neuron, row_begin, nrows, dmin=0.10, dmax=0.25):
    out = np.empty((nrows, neuron), dtype=np.float32)
    _lib.orc_gen_features(seed, neuron, row_begin, nrows, dmin, dmax, out)
    return out


def feature_threshold(seed, row, dmin=0.10, dmax=0.25):
    return int(_lib.orc_feature_threshold(seed, row, dmin, dmax))


def hash_reorder(v, buckets, domain):
    return int(_lib.orc_hash_reorder(v, buckets, domain))


def read_weight_tsv(path, begin_idx=1):
    """Returns (row, col, val, n_rows, n_cols): row = output neuron, col = input neuron."""
    n = _lib.orc_count_tsv_triples(path.encode())
    if n < 0:
        raise FileNotFoundError(path)
    row = np.empty(max(n, 1), dtype=np.int32)
    col = np.empty(max(n, 1), dtype=np.int32)
    val = np.empty(max(n, 1), dtype=np.float32)
    nr, nc = C.c_int(), C.c_int()
    got = _lib.orc_read_weight_tsv(path.encode(), begin_idx, n, row, col, val, C.byref(nr), C.byref(nc))
    assert got == n
    return row[:n].copy(), col[:n].copy(), val[:n].copy(), nr.value, nc.value


def coo_to_csr(row, col, val, n_rows):
    row = np.ascontiguousarray(row, dtype=np.int32)
    col = np.ascontiguousarray(col, dtype=np.int32)
    val = np.ascontiguousarray(val, dtype=np.float32)
    nnz = len(row)
    rowptr = np.empty(n_rows + 1, dtype=np.int32)
    ccol = np.empty(max(nnz, 1), dtype=np.int32)
    cval = np.empty(max(nnz, 1), dtype=np.float32)
    rc = _lib.orc_coo_to_csr(nnz, n_rows, row if nnz else np.zeros(1, np.int32),
                             col if nnz else np.zeros(1, np.int32),
                             val if nnz else np.zeros(1, np.float32), rowptr, ccol, cval)
    if rc != 0:
        raise ValueError("orc_coo_to_csr failed: %d" % rc)
    return rowptr, ccol[:nnz].copy(), cval[:nnz].copy()


def read_features_tsv(path, neuron, batch):
    dense = np.zeros((batch, neuron), dtype=np.float32)
    kept = _lib.orc_read_features_tsv(path.encode(), neuron, batch, dense)
    if kept < 0:
        raise FileNotFoundError(path)
    return dense, int(kept)


def read_weights_bin(path, neuron, layer, nnz=None):
    """Layer record `layer` of a packed "neuron<N>.bin" as CSR (rowptr, col, val), following readweights
    of the reference's library benchmark (benchmark/cusparse/cusparse.cu:318-358): int32 row[nnz],
    int32 col[nnz], float32 val[nnz] per layer, 1-based; CSR row = row-1 (the output neuron of
    C = A*B there, cusparse.cu:118-150), CSR column = col-1, entries of a row in file order."""
    nnz = 32 * neuron if nnz is None else nnz
    with open(path, "rb") as f:
        f.seek(12 * nnz * layer)
        row = np.fromfile(f, dtype="<i4", count=nnz)
        col = np.fromfile(f, dtype="<i4", count=nnz)
        val = np.fromfile(f, dtype="<f4", count=nnz)
    if len(val) != nnz:
        raise IOError("short read")
    order = np.argsort(row, kind="stable")
    rowptr = np.zeros(neuron + 1, dtype=np.int32)
    np.cumsum(np.bincount(row - 1, minlength=neuron), out=rowptr[1:])
    return rowptr, (col[order] - 1).astype(np.int32), val[order].astype(np.float32)


def read_features_bin(path, neuron, batch):
    """Dense batch x neuron features from a packed "sparse-images-<N>.bin" (readinput,
    benchmark/cusparse/cusparse.cu:361-383): int32 row[] = neuron, int32 col[] = image,
    float32 val[]; images beyond `batch` are skipped."""
    raw = np.fromfile(path, dtype="<i4")
    n = len(raw) // 3
    row, col = raw[:n], raw[n:2 * n]
    val = raw[2 * n:3 * n].view("<f4")
    dense = np.zeros((batch, neuron), dtype=np.float32)
    for e in range(n):                      # file order: a later duplicate overwrites an earlier one
        if col[e] - 1 < batch:
            dense[col[e] - 1, row[e] - 1] = val[e]
    return dense


def relu_clamp(x):
    return float(_lib.orc_relu_clamp(C.c_float(x)))


def layer(yin, csr, bias):
    """One layer on row-major `yin`; returns (yout, active int32[nrows])."""
    rowptr, col, val = csr
    yin = np.ascontiguousarray(yin, dtype=np.float32)
    nrows, neuron = yin.shape
    yout = np.empty_like(yin)
    active = np.zeros(max(nrows, 1), dtype=np.int32)
    if nrows:
        _lib.orc_layer(yin, nrows, neuron, np.ascontiguousarray(rowptr, np.int32),
                       np.ascontiguousarray(col, np.int32) if len(col) else np.zeros(1, np.int32),
                       np.ascontiguousarray(val, np.float32) if len(val) else np.zeros(1, np.float32),
                       bias, yout, active)
    return yout, active[:nrows]


def compact(y, active, gid):
    y = np.ascontiguousarray(y, dtype=np.float32)
    nrows, neuron = y.shape
    out = np.empty_like(y)
    gout = np.empty(max(nrows, 1), dtype=np.int32)
    n = _lib.orc_compact(y, nrows, neuron, np.ascontiguousarray(active, np.int32) if nrows else np.zeros(1, np.int32),
                         np.ascontiguousarray(gid, np.int32) if nrows else np.zeros(1, np.int32), out, gout) if nrows else 0
    return out[:n].copy(), gout[:n].copy()


def infer(features, layers, bias, prune=True, keep=None):
    """Layer chain.  `layers` is a sequence of CSR triples (or a callable l -> CSR).

    Returns a dict with, per layer, the global ids of the rows that are active after it
    ('active_ids'), the final activations of the rows still carried ('y', with their global ids
    in 'gid'), and - when `keep` is a collection of layer numbers - a copy of (gid, y) after
    each of those layers in 'kept'.  With prune=False every row is carried to the end.
    """
    y = np.ascontiguousarray(features, dtype=np.float32)
    gid = np.arange(y.shape[0], dtype=np.int32)
    n_layers = len(layers) if hasattr(layers, "__len__") else None
    active_ids, kept = [], {}
    l = 0
    while n_layers is None or l < n_layers:
        csr = layers[l] if n_layers is not None else layers(l)
        if csr is None:
            break
        y, act = layer(y, csr, bias)
        active_ids.append(gid[act != 0].copy())
        if prune:
            y, gid = compact(y, act, gid)
        if keep is not None and l in keep:
            kept[l] = (gid.copy(), y.copy())
        l += 1
    return {"active_ids": active_ids, "y": y, "gid": gid, "kept": kept,
            "categories": active_ids[-1] if active_ids else gid}


def receptive_field(layers, out_neurons):
    """Input neurons of layers[0] that the output neurons `out_neurons` of layers[-1] depend on
    (ascending): the reference's FuseLayer, one orc_need_access step per layer from the last back."""
    neuron = len(layers[-1][0]) - 1
    flags = np.zeros(neuron, np.uint8)
    flags[np.asarray(out_neurons, dtype=np.int64)] = 1
    for rowptr, col, _ in reversed(list(layers)):
        nxt = np.zeros(neuron, np.uint8)
        _lib.orc_need_access(neuron, np.ascontiguousarray(rowptr, np.int32), np.ascontiguousarray(col, np.int32), flags, nxt)
        flags = nxt
    return np.nonzero(flags)[0].astype(np.int32)
