"""The CPU oracle against the reference's own CPU code (oracle/_ref/ref_check, built from the
reference's headers where the reference is mounted) and against the committed fixtures."""
import json
import os
import subprocess

import numpy as np
import pytest

from helpers import random_csr, sort_rows

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = os.path.join(HERE, "golden")


def _ref(orc):
    if not os.path.exists(orc.REF_CHECK) and os.path.isdir("/root/reference/src/utils"):
        orc.build(with_ref=True)   # a fresh checkout beside the mounted reference: build the harness once
    if not os.path.exists(orc.REF_CHECK):
        pytest.skip("oracle/_ref/ref_check not built (the reference is not mounted here)")
    return orc.REF_CHECK


def _write_tsv(path, csr, rng=None):
    rowptr, col, val = csr
    lines = ["%d\t%d\t%.9g\n" % (col[e] + 1, j + 1, val[e]) for j in range(len(rowptr) - 1)
             for e in range(rowptr[j], rowptr[j + 1])]
    if rng is not None:
        rng.shuffle(lines)
    with open(path, "w") as f:
        f.writelines(lines)


def test_weight_loader_matches_reference_coomatrix(orc, tmp_path):
    """Orientation ("in out value" -> row = out-1, col = in-1), dimensions and the
    (row, col)-sorted order of the reference's COOMatrix, element by element."""
    ref = _ref(orc)
    rng = np.random.default_rng(1)
    csr = sort_rows(random_csr(rng, 48, rng.integers(1, 9, size=48), "general"))
    p = str(tmp_path / "w.tsv")
    _write_tsv(p, csr, rng)
    out = subprocess.run([ref, "coo", p], capture_output=True, text=True, check=True).stdout.split("\n")
    nr, nc, nnz = map(int, out[0].split())
    row, col, val, onr, onc = orc.read_weight_tsv(p)
    assert (nr, nc, nnz) == (onr, onc, len(row))
    rowptr, ccol, cval = orc.coo_to_csr(row, col, val, nr)
    got = [(j, int(ccol[e]), float(cval[e])) for j in range(nr) for e in range(rowptr[j], rowptr[j + 1])]
    want = [(int(a), int(b), float(np.float32(float(c)))) for a, b, c in (ln.split() for ln in out[1:1 + nnz])]
    assert got == want
    # and the loader reproduces the layer that was written
    assert np.array_equal(rowptr[:len(csr[0])], csr[0][:len(rowptr)])
    assert np.array_equal(ccol, csr[1]) and np.array_equal(cval, csr[2])


@pytest.mark.parametrize("buckets,domain", [(64, 1024), (256, 4096), (4, 64)])
def test_hash_reorder_matches_reference(orc, buckets, domain):
    ref = _ref(orc)
    out = subprocess.run([ref, "hash", str(buckets), str(domain)], capture_output=True, text=True, check=True).stdout
    want = [int(x) for x in out.split()]
    got = [orc.hash_reorder(v, buckets, domain) for v in range(domain)]
    assert got == want


def test_single_layer_accepted_by_reference_cpuspmm(orc, tmp_path):
    """CpuSpmm::run_and_cmp accepts the oracle's layer output (no bias, nothing clamped) and
    rejects it after a perturbation or a transposition mistake."""
    ref = _ref(orc)
    rng = np.random.default_rng(2)
    n, b = 96, 7
    csr = sort_rows(random_csr(rng, n, 8, "uniform"))
    wp = str(tmp_path / "w.tsv")
    _write_tsv(wp, csr, rng)
    x = rng.uniform(0, 8, size=(b, n)).astype(np.float32)
    y, _ = orc.layer(x, csr, 0.0)
    assert y.max() < 32  # the reference comparator has no clamp
    x.tofile(str(tmp_path / "in.f32"))

    def run(arr):
        arr.astype("<f4").tofile(str(tmp_path / "out.f32"))
        return subprocess.run([ref, "spmm", wp, str(n), str(b), str(tmp_path / "in.f32"), str(tmp_path / "out.f32")],
                              capture_output=True, text=True)
    ok = run(y)
    assert ok.returncode == 0 and "[Success]" in ok.stdout
    bad = y.copy()
    bad[3, 17] += 0.01
    assert run(bad).returncode != 0
    # a transposed weight matrix is a different answer, and the reference notices
    rowptr, col, val = csr
    rows = np.repeat(np.arange(n, dtype=np.int32), np.diff(rowptr))
    yt, _ = orc.layer(x, orc.coo_to_csr(col, rows, val, n), 0.0)
    assert run(yt).returncode != 0


@pytest.mark.parametrize("ibias", [0, -1, -3])
def test_chain_accepted_by_reference_cpuspmmfuse(orc, tmp_path, ibias):
    """Three chained layers with bias and clamp against CpuSpmmFuse::run_and_cmp (integer bias,
    which is exact here)."""
    ref = _ref(orc)
    rng = np.random.default_rng(3)
    n, b = 64, 9
    layers = [sort_rows(random_csr(rng, n, 8, "pow2")) for _ in range(3)]
    paths = []
    for i, csr in enumerate(layers):
        paths.append(str(tmp_path / ("w%d.tsv" % i)))
        _write_tsv(paths[-1], csr, rng)
    x = rng.uniform(0, 32, size=(b, n)).astype(np.float32)
    x.tofile(str(tmp_path / "in.f32"))
    r = orc.infer(x, layers, float(ibias), prune=False)
    y = r["y"]
    assert (y == 0).any() and (y > 0).any()  # both branches of the clamp are exercised
    y.astype("<f4").tofile(str(tmp_path / "out.f32"))
    ok = subprocess.run([ref, "fuse", str(n), str(b), str(ibias), str(tmp_path / "in.f32"),
                         str(tmp_path / "out.f32")] + paths, capture_output=True, text=True)
    assert ok.returncode == 0 and "[Success]" in ok.stdout, ok.stdout + ok.stderr
    # dropping the bias is caught
    if ibias != 0:
        orc.infer(x, layers, 0.0, prune=False)["y"].astype("<f4").tofile(str(tmp_path / "out.f32"))
        bad = subprocess.run([ref, "fuse", str(n), str(b), str(ibias), str(tmp_path / "in.f32"),
                              str(tmp_path / "out.f32")] + paths, capture_output=True, text=True)
        assert bad.returncode != 0


def test_compaction_accepted_by_reference_transpose_delete(orc, tmp_path):
    """The oracle's stable compaction against CpuTransposeDelete::run_and_cmp (the reference's
    check of its transpose-and-delete step)."""
    ref = _ref(orc)
    rng = np.random.default_rng(4)
    n, b = 32, 40
    y = rng.uniform(0, 5, size=(b, n)).astype(np.float32)
    active = (rng.random(b) < 0.5).astype(np.int32)
    out, gid = orc.compact(y, active, np.arange(b, dtype=np.int32))
    old_to_new = np.full(b, -1, np.int32)
    old_to_new[gid] = np.arange(len(gid))
    y.T.copy().astype("<f4").tofile(str(tmp_path / "in.f32"))
    old_to_new.astype("<i4").tofile(str(tmp_path / "map.i32"))
    out.astype("<f4").tofile(str(tmp_path / "out.f32"))
    ok = subprocess.run([ref, "transpose_delete", str(n), str(b), str(len(gid)), str(tmp_path / "in.f32"),
                         str(tmp_path / "map.i32"), str(tmp_path / "out.f32")], capture_output=True, text=True)
    assert ok.returncode == 0 and "[Success]" in ok.stdout


def test_receptive_field_matches_reference_fuselayer(orc, tmp_path):
    """orc_need_access against ftxj::FuseLayer (src/fuse/fuse.h): blocks of 16 output neurons of the
    last layer through one, two and three layers - the committed 64-neuron fixtures and random layers."""
    ref = _ref(orc)
    rng = np.random.default_rng(9)
    n = 64
    fixture = [os.path.join(GOLD, "tiny_n64-l%d.tsv" % l) for l in (1, 2)]
    layers = []
    for f in fixture:
        r, c, v, nr, nc = orc.read_weight_tsv(f)
        layers.append(orc.coo_to_csr(r, c, v, n))
    extra = random_csr(rng, n, rng.integers(1, 6, size=n), "general")
    path3 = str(tmp_path / "extra.tsv")
    _write_tsv(path3, extra, rng)
    chain = [(layers + [extra], fixture + [path3]), (layers, fixture), ([extra], [path3])]
    for lays, files in chain:
        # FuseLayer starts from the LAST layer and fuses the earlier ones in turn
        out = subprocess.run([ref, "need_access", "16"] + files[::-1], check=True, capture_output=True, text=True).stdout
        blocks = [ln for ln in out.splitlines() if ln.startswith("block b = ")]
        assert len(blocks) == n // 16
        for b, ln in enumerate(blocks):
            head, _, tail = ln.partition(" : ")
            want = [int(x) for x in tail.split(",") if x.strip()]
            assert "size = %d" % len(want) in head
            got = orc.receptive_field(lays, range(16 * b, 16 * b + 16))
            assert got.tolist() == want


def test_oracle_reproduces_committed_fixtures(orc):
    """tests/golden/: TSV layers + features -> expected activations / categories (confirmed by the
    reference's comparators when the fixture was generated)."""
    exp = json.load(open(os.path.join(GOLD, "tiny_expected.json")))
    N, B = 64, 12
    layers = []
    for l in (1, 2):
        row, col, val, nr, nc = orc.read_weight_tsv(os.path.join(GOLD, "tiny_n64-l%d.tsv" % l))
        assert (nr, nc) == (N, N)
        layers.append(orc.coo_to_csr(row, col, val, N))
    feats, kept = orc.read_features_tsv(os.path.join(GOLD, "tiny_features-64.tsv"), N, B)
    assert not feats[3].any() and (feats[7] == 32).all()
    for bias in (0.0, -1.0, -0.3):
        e = exp["bias_%g" % bias]
        r = orc.infer(feats, layers, bias, prune=False, keep={0, 1})
        assert [a.tolist() for a in r["active_ids"]] == e["active_ids"]
        assert r["kept"][0][1].astype("<f4").tobytes().hex() == e["y_layer1_hex"]
        assert r["kept"][1][1].astype("<f4").tobytes().hex() == e["y_layer2_hex"]
