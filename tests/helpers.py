"""Shared helpers of the parity tests."""
import numpy as np


def random_csr(rng, n, row_nnz, values="pow2"):
    """Random square layer in CSR (row = output neuron): row j holds row_nnz[j] distinct inputs."""
    rowptr = np.zeros(n + 1, np.int32)
    cols, vals = [], []
    for j in range(n):
        k = int(row_nnz[j]) if hasattr(row_nnz, "__len__") else int(row_nnz)
        c = rng.choice(n, size=k, replace=False)
        rng.shuffle(c)  # unsorted on purpose: the library must sort
        cols.append(c)
        if values == "pow2":
            v = np.ldexp(1.0, rng.integers(-6, 1, size=k)) * rng.choice([-1.0, 1.0], size=k)
        elif values == "uniform":
            v = np.full(k, 0.0625)
        else:
            v = rng.uniform(-0.2, 0.3, size=k)
        vals.append(v.astype(np.float32))
        rowptr[j + 1] = rowptr[j] + k
    col = np.concatenate(cols).astype(np.int32) if cols else np.zeros(0, np.int32)
    val = np.concatenate(vals).astype(np.float32) if vals else np.zeros(0, np.float32)
    return rowptr, col, val


def sort_rows(csr):
    """The same layer with every row sorted by input index (stable)."""
    rowptr, col, val = csr
    col2, val2 = col.copy(), val.copy()
    for j in range(len(rowptr) - 1):
        b, e = rowptr[j], rowptr[j + 1]
        o = np.argsort(col[b:e], kind="stable")
        col2[b:e] = col[b:e][o]
        val2[b:e] = val[b:e][o]
    return rowptr, col2, val2


def same_floats(a, b):
    """Bit-for-bit equality of fp32 arrays, except that +0.0 and -0.0 count as equal."""
    a = np.asarray(a, np.float32)
    b = np.asarray(b, np.float32)
    return a.shape == b.shape and bool(np.all((a == b) | (np.isnan(a) & np.isnan(b))))


def radix_like_csr(rng, n, stride, values="uniform", relabel=True, run=16, perm=None):
    """RadiX-Net-like layer: the outputs of group g (16 consecutive outputs) all read the two
    16-wide input runs [16g, 16g+16) and [16g+stride, 16g+stride+16) (mod n) - the structure the
    reference's kernels assume after its hash reorder - optionally hidden behind random
    relabellings of inputs and outputs, as in the raw challenge files.  perm: one relabelling for
    inputs and outputs alike (the layers of a network built with the same perm share a neuron
    numbering, as consecutive layer files of the challenge do)."""
    pin = perm if perm is not None else rng.permutation(n) if relabel else np.arange(n)
    pout = perm if perm is not None else rng.permutation(n) if relabel else np.arange(n)
    rows = [None] * n
    for j in range(n):
        g = j // run
        ins = np.concatenate([np.arange(run * g, run * g + run), np.arange(run * g + stride, run * g + stride + run)]) % n
        rows[pout[j]] = np.unique(pin[ins])
    rowptr = np.zeros(n + 1, np.int32)
    for j in range(n):
        rowptr[j + 1] = rowptr[j] + len(rows[j])
    col = np.concatenate(rows).astype(np.int32)
    k = len(col)
    if values == "uniform":
        val = np.full(k, 0.0625, np.float32)
    elif values == "pow2":
        val = (np.ldexp(1.0, rng.integers(-6, -2, size=k)) * rng.choice([-1.0, 1.0], size=k)).astype(np.float32)
    else:
        val = rng.uniform(-0.1, 0.15, size=k).astype(np.float32)
    return rowptr, col, val


def hub_block_csr(rng, n, values="uniform"):
    """Groups of 16 outputs that read their own 16-wide input run plus the shared run [0, 16):
    identical rows inside a group, but no chain of groups (one run is read by every group)."""
    pin, pout = rng.permutation(n), rng.permutation(n)
    rows = [None] * n
    for j in range(n):
        g = j // 16
        rows[pout[j]] = np.unique(pin[np.concatenate([np.arange(16), np.arange(16 * g, 16 * g + 16)])])
    rowptr = np.zeros(n + 1, np.int32)
    rowptr[1:] = np.cumsum([len(r) for r in rows])
    col = np.concatenate(rows).astype(np.int32)
    k = len(col)
    if values == "uniform":
        val = np.full(k, 0.0625, np.float32)
    elif values == "pow2":
        val = (np.ldexp(1.0, rng.integers(-6, -2, size=k)) * rng.choice([-1.0, 1.0], size=k)).astype(np.float32)
    else:
        val = rng.uniform(-0.1, 0.15, size=k).astype(np.float32)
    return rowptr, col, val


def common_band_csr(rng, n, perm, values="uniform", k=32):
    """A convolution-like layer over a neuron order common to all layers of a network: the neuron at
    place t of the order (neuron perm[t]) reads the neurons at places t-k+1 .. t (mod n).  With a
    random `perm` the band is hidden; consecutive layers built over the same `perm` write their
    outputs where the next one's band reads them."""
    rows = [None] * n
    for t in range(n):
        rows[perm[t]] = np.sort(perm[(t - np.arange(k)) % n])
    rowptr = np.arange(n + 1, dtype=np.int32) * k
    col = np.concatenate(rows).astype(np.int32)
    m = len(col)
    if values == "uniform":
        val = np.full(m, 0.0625, np.float32)
    elif values == "pow2":
        val = (np.ldexp(1.0, rng.integers(-5, -2, size=m)) * rng.choice([-1.0, 1.0], size=m, p=[0.1, 0.9])).astype(np.float32)
    else:
        val = rng.uniform(-0.05, 0.15, size=m).astype(np.float32)
    return rowptr, col, val
