#!/usr/bin/env python3
"""Writes the small committed fixtures under tests/golden/.

Run from the repository root in a container that has the reference mounted:

    python tests/golden/make_fixtures.py

The fixtures are DATA: two tiny weight layers and a feature matrix in the challenge's TSV
formats, plus the expected activations / categories computed by the CPU oracle.  Before
anything is written the expected values are confirmed by the reference's own CPU comparators
through oracle/_ref/ref_check (CpuSpmm for layer 1 without epilogue, CpuSpmmFuse with an
integer bias for the two-layer chain), so a fixture cannot be generated from an oracle that
disagrees with the reference.  Also records hashes of generated buffers (generator pinning).
"""
import hashlib
import json
import os
import subprocess
import sys
import tempfile

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import oracle as orc  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
N, B, K = 64, 12, 8


def write_weight_tsv(path, csr, rng):
    rowptr, col, val = csr
    lines = []
    for j in range(len(rowptr) - 1):
        for e in range(rowptr[j], rowptr[j + 1]):
            lines.append("%d\t%d\t%.9g\n" % (col[e] + 1, j + 1, val[e]))  # "in out value", 1-based
    rng.shuffle(lines)  # the loaders must not depend on file order
    with open(path, "w") as f:
        f.writelines(lines)


def main():
    rng = np.random.default_rng(2021)
    layers = []
    for l in range(2):
        rowptr, col, val = orc.gen_layer_csr(77, l, N, K, 0.0625)
        val = rng.choice(np.array([0.0625, 0.125, 0.25, -0.125, 0.5], np.float32), size=len(val)).astype(np.float32)
        layers.append((rowptr, col, val))
        write_weight_tsv(os.path.join(HERE, "tiny_n64-l%d.tsv" % (l + 1)), layers[-1], rng)
    feats = (rng.integers(0, 9, size=(B, N)) * (rng.random((B, N)) < 0.4)).astype(np.float32)
    feats[3] = 0.0            # an all-zero row
    feats[7] = 32.0           # a saturated row
    with open(os.path.join(HERE, "tiny_features-64.tsv"), "w") as f:
        for b in range(B + 2):  # two rows beyond the batch, which the loaders must skip
            src = feats[b % B]
            for n in range(N):
                if src[n] != 0:
                    f.write("%d\t%d\t%.9g\n" % (b + 1, n + 1, src[n]))

    expected = {}
    for bias in (0.0, -1.0, -0.3):
        r = orc.infer(feats, layers, bias, prune=False, keep={0, 1})
        expected["bias_%g" % bias] = {
            "active_ids": [a.tolist() for a in r["active_ids"]],
            "y_layer1_hex": r["kept"][0][1].astype("<f4").tobytes().hex(),
            "y_layer2_hex": r["kept"][1][1].astype("<f4").tobytes().hex(),
        }

    # confirm with the reference's comparators before writing
    ref = orc.REF_CHECK
    if not os.path.exists(ref):
        raise SystemExit("oracle/_ref/ref_check is missing: run `make -C oracle` with the reference mounted")
    with tempfile.TemporaryDirectory() as td:
        fin = os.path.join(td, "in.f32")
        feats.astype("<f4").tofile(fin)
        for bias in (0, -1):
            r = orc.infer(feats, layers, float(bias), prune=False, keep={0, 1})
            fout = os.path.join(td, "out.f32")
            r["kept"][1][1].astype("<f4").tofile(fout)
            out = subprocess.run([ref, "fuse", str(N), str(B), str(bias), fin, fout,
                                  os.path.join(HERE, "tiny_n64-l1.tsv"), os.path.join(HERE, "tiny_n64-l2.tsv")],
                                 capture_output=True, text=True)
            assert out.returncode == 0 and "[Success]" in out.stdout, out.stdout + out.stderr

    # generator pinning: hashes of generated buffers
    gen = {}
    for (seed, layer, n) in [(0, 0, 1024), (0, 119, 1024), (5, 3, 4096)]:
        rowptr, col, val = orc.gen_layer_csr(seed, layer, n)
        perm, o, s = orc.gen_layer_params(seed, layer, n)
        gen["layer_seed%d_l%d_n%d" % (seed, layer, n)] = {
            "col_sha256": hashlib.sha256(col.astype("<i4").tobytes()).hexdigest(), "offset": o, "stride": s,
            "perm_head": perm[:8].tolist()}
    for (seed, n, r0, nr) in [(0, 1024, 0, 64), (0, 65536, 59990, 4)]:
        f = orc.gen_features(seed, n, r0, nr)
        gen["features_seed%d_n%d_r%d_%d" % (seed, n, r0, nr)] = {
            "sha256": hashlib.sha256(f.astype("<f4").tobytes()).hexdigest(), "nnz": int(f.sum())}
    expected["generator"] = gen
    expected["splitmix64_of_0"] = orc.splitmix64(0)
    with open(os.path.join(HERE, "tiny_expected.json"), "w") as f:
        json.dump(expected, f, indent=1)
    print("fixtures written to", HERE)


if __name__ == "__main__":
    main()
