"""What the mathematics fixes about the oracle: closed forms, special values, invariants.
Each check is chosen so that a plausible mistake (transposed operand, wrong order, fused
multiply-add, bias before the sum, unstable compaction) fails it."""
import math

import numpy as np
import pytest

from helpers import random_csr, sort_rows


def _csr_from_dense(w):
    """w[out, in] dense -> CSR (row = output)."""
    n = w.shape[0]
    rowptr = np.zeros(n + 1, np.int32)
    col, val = [], []
    for j in range(n):
        nz = np.nonzero(w[j])[0]
        col.extend(nz.tolist())
        val.extend(w[j, nz].tolist())
        rowptr[j + 1] = len(col)
    return rowptr, np.array(col, np.int32), np.array(val, np.float32)


def test_dense_brute_force(orc):
    rng = np.random.default_rng(0)
    n, b = 48, 10
    w = (rng.random((n, n)) < 0.2) * rng.uniform(-1, 1, size=(n, n))
    w = w.astype(np.float32)
    x = rng.uniform(0, 3, size=(b, n)).astype(np.float32)
    y, act = orc.layer(x, _csr_from_dense(w), -0.25)
    want = np.clip(x.astype(np.float64) @ w.astype(np.float64).T - 0.25, 0, 32)
    assert np.allclose(y, want, rtol=1e-5, atol=1e-5)
    assert np.array_equal(act != 0, (y != 0).any(axis=1))


def test_permutation_matrix_moves_columns(orc):
    rng = np.random.default_rng(1)
    n, b = 40, 5
    perm = rng.permutation(n)            # output j reads input perm[j]
    w = np.zeros((n, n), np.float32)
    w[np.arange(n), perm] = 1.0
    x = rng.uniform(0, 30, size=(b, n)).astype(np.float32)
    y, _ = orc.layer(x, _csr_from_dense(w), 0.0)
    assert np.array_equal(y, x[:, perm])


def test_tsv_orientation_closed_form(orc, tmp_path):
    """Line "a b v" means W(a, b) = v with Y_out[:, b] += Y_in[:, a] * v."""
    p = tmp_path / "w.tsv"
    p.write_text("1\t3\t2.0\n2\t3\t0.5\n3\t1\t1.0\n")
    row, col, val, nr, nc = orc.read_weight_tsv(str(p))
    csr = orc.coo_to_csr(row, col, val, 3)
    x = np.array([[1.0, 10.0, 100.0]], np.float32)
    y, _ = orc.layer(x, csr, 0.0)
    assert y.tolist() == [[32.0, 0.0, 7.0]]   # out1 = in3 (clamped at 32), out2 = 0, out3 = 2*1 + 0.5*10


def test_features_tsv_known_answer(orc, tmp_path):
    p = tmp_path / "f.tsv"
    p.write_text("1\t2\t1\n3\t1\t1\n2\t4\t0.5\n4\t1\t1\n")  # row 4 is beyond batch 3
    dense, kept = orc.read_features_tsv(str(p), 4, 3)
    assert kept == 3
    assert dense.tolist() == [[0, 1, 0, 0], [0, 0, 0, 0.5], [1, 0, 0, 0]]


def test_all_ones_input(orc):
    csr = orc.gen_layer_csr(0, 0, 1024)
    y, act = orc.layer(np.ones((2, 1024), np.float32), csr, -0.3)
    assert (y == np.float32(np.float32(2.0) + np.float32(-0.3))).all() and act.all()


@pytest.mark.parametrize("x,want", [(-0.0, -0.0), (0.0, 0.0), (-1e-30, 0.0), (1e-30, 1e-30), (32.0, 32.0),
                                     (np.nextafter(np.float32(32), np.float32(64)), 32.0), (1e30, 32.0),
                                     (-1e30, 0.0), (31.999998, 31.999998)])
def test_relu_clamp_special_values(orc, x, want):
    got = orc.relu_clamp(x)
    assert got == np.float32(want) and math.copysign(1, got) == math.copysign(1, np.float32(want))


def test_relu_clamp_nan_passes_through(orc):
    assert math.isnan(orc.relu_clamp(float("nan")))


def test_threshold_row_is_inactive(orc):
    """y = -bias exactly gives 0 and an inactive row; one ulp above gives an active row."""
    w = np.zeros((2, 2), np.float32)
    w[0, 0] = 1.0
    w[1, 1] = 1.0
    csr = _csr_from_dense(w)
    x = np.array([[0.5, 0.25], [np.nextafter(np.float32(0.5), np.float32(1)), 0.0]], np.float32)
    y, act = orc.layer(x, csr, -0.5)
    assert y[0].tolist() == [0.0, 0.0] and act.tolist() == [0, 1] and y[1, 0] > 0


def test_accumulation_order_is_ascending_input_index(orc):
    """fp32: (1e8 + 1) - 1e8 = 0 but (1e8 - 1e8) + 1 = 1."""
    w = np.zeros((3, 3), np.float32)
    w[0, :] = 1.0
    y, _ = orc.layer(np.array([[1e8, 1.0, -1e8]], np.float32), _csr_from_dense(w), 0.0)
    assert y[0, 0] == 0.0
    y, _ = orc.layer(np.array([[1e8, -1e8, 1.0]], np.float32), _csr_from_dense(w), 0.0)
    assert y[0, 0] == 1.0


def test_bias_is_added_after_the_sum(orc):
    """acc starting at bias would round differently: 1e8 + (-0.5) is 1e8, then - 1e8 gives 0;
    sum first gives exactly 0, then + (-0.5) clamps to 0 as well - so use a positive bias."""
    w = np.zeros((2, 2), np.float32)
    w[0, :] = 1.0
    y, _ = orc.layer(np.array([[1e8, -1e8]], np.float32), _csr_from_dense(w), 0.75)
    assert y[0, 0] == 0.75


def test_multiply_then_add_is_not_fused(orc):
    """x*w rounds to 1 + 2^-11 (tie to even); a fused multiply-add would keep the 2^-24."""
    a = np.float32(1 + 2.0 ** -12)
    w = np.zeros((2, 2), np.float32)
    w[0, 0] = -1.0
    w[0, 1] = a
    x = np.array([[np.float32(1 + 2.0 ** -11), a]], np.float32)
    y, _ = orc.layer(x, _csr_from_dense(w), 0.0)
    assert y[0, 0] == 0.0


def test_chain_fixed_points(orc):
    layers = [orc.gen_layer_csr(1, l, 1024) for l in range(6)]
    x = np.zeros((3, 1024), np.float32)
    x[1] = 32.0
    x[2] = 1.0
    r = orc.infer(x, layers, -0.3, prune=False, keep={0})
    y1 = r["kept"][0][1]
    assert not y1[0].any()                       # zero row stays zero when bias < 0
    assert (y1[1] == 32.0).all()                 # saturated row: min(64 - 0.3, 32)
    assert (y1[2] == np.float32(np.float32(2.0) - np.float32(0.3))).all()   # constant row c -> 2c + bias
    assert r["active_ids"][-1].tolist() == [1, 2]
    assert (r["y"][1] == 32.0).all() and (r["y"][2] == 32.0).all()


def test_pruning_invariants(orc):
    N, B, L = 1024, 400, 10
    layers = [orc.gen_layer_csr(4, l, N) for l in range(L)]
    feats = orc.gen_features(4, N, 0, B, 0.10, 0.50)
    full = orc.infer(feats, layers, -0.3, prune=False)
    pruned = orc.infer(feats, layers, -0.3, prune=True)
    counts = [len(a) for a in pruned["active_ids"]]
    assert counts == sorted(counts, reverse=True) and 0 < counts[-1] < B   # non-increasing, non-trivial
    for a, b in zip(full["active_ids"], pruned["active_ids"]):
        assert np.array_equal(a, b)
    assert np.array_equal(pruned["gid"], np.sort(pruned["gid"]))           # stable: order preserved
    assert np.array_equal(pruned["y"], full["y"][pruned["gid"]])           # same values on survivors
    # row independence: a subset run equals the full run restricted to the subset
    sub = np.arange(17, B, 3)
    part = orc.infer(feats[sub], layers, -0.3, prune=False)
    assert np.array_equal(part["y"], full["y"][sub])


def test_unsorted_rows_are_sorted_by_loader(orc):
    rng = np.random.default_rng(5)
    csr = random_csr(rng, 32, 6, "general")
    rowptr, col, val = csr
    rows = np.repeat(np.arange(32, dtype=np.int32), np.diff(rowptr))
    got = orc.coo_to_csr(rows, col, val, 32)
    want = sort_rows(csr)
    assert all(np.array_equal(a, b) for a, b in zip(got, want))


def test_receptive_field_against_boolean_matrix_products(orc):
    """FuseLayer's analysis is reachability through the layers' patterns: compare with dense
    boolean products of the transposed patterns, and with what a band fixes in closed form."""
    rng = np.random.default_rng(5)
    n = 48
    layers = [random_csr(rng, n, rng.integers(0, 5, size=n), "general") for _ in range(3)]
    dense = []
    for rowptr, col, _ in layers:
        m = np.zeros((n, n), bool)          # m[out, in]
        for j in range(n):
            m[j, col[rowptr[j]:rowptr[j + 1]]] = True
        dense.append(m)
    for outs in ([0], [3, 4, 5, 6], list(range(16, 32)), []):
        need = np.zeros(n, bool)
        need[outs] = True
        for depth in (1, 2, 3):
            v = need.copy()
            for m in reversed(dense[3 - depth:]):
                v = (m & v[:, None]).any(axis=0)
            got = orc.receptive_field(layers[3 - depth:], outs)
            assert np.array_equal(got, np.nonzero(v)[0])
    # a band of width 8 in natural order: a tile of T outputs needs T+7 inputs through one layer,
    # T+14 through two, and the set is the tile's places shifted back
    n, k, t0, T = 64, 8, 20, 10
    rowptr = np.arange(n + 1, dtype=np.int32) * k
    col = np.sort((np.arange(n)[:, None] - np.arange(k)[None, :]) % n, axis=1).reshape(-1).astype(np.int32)
    band = (rowptr, col, np.ones(n * k, np.float32))
    assert np.array_equal(orc.receptive_field([band], range(t0, t0 + T)), np.arange(t0 - 7, t0 + T))
    assert np.array_equal(orc.receptive_field([band, band], range(t0, t0 + T)), np.arange(t0 - 14, t0 + T))
    # a permutation matrix moves the block, whatever its size
    perm = rng.permutation(n).astype(np.int32)
    pm = (np.arange(n + 1, dtype=np.int32), perm, np.ones(n, np.float32))
    assert np.array_equal(orc.receptive_field([pm], [1, 2, 3]), np.sort(perm[[1, 2, 3]]))
