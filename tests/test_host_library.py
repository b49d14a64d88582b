"""Host side of the C-ABI library, without a GPU: the library loads and exports every symbol
the header declares, the inspector's plans reproduce the oracle when emulated on the CPU, the
loaders and the error paths behave as documented."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from helpers import common_band_csr, hub_block_csr, radix_like_csr, random_csr, same_floats, sort_rows

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLD = os.path.join(ROOT, "tests", "golden")


def test_library_exports_every_declared_symbol(gc):
    header = open(os.path.join(ROOT, "include", "spdnn.h")).read()
    names = sorted(set(re.findall(r"\b(spdnn_[a-z0-9_]+)\s*\(", header)))
    assert len(names) >= 30
    lib = ctypes.CDLL(gc.lib_path())
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing
    assert gc.load_library().spdnn_version() >= 100


def test_reference_tables(gc):
    # bias by neuron count (reference src/network.cpp:73-78)
    assert [gc.reference_bias(n) for n in (1024, 4096, 16384, 65536)] == pytest.approx([-0.3, -0.35, -0.4, -0.45])
    with pytest.raises(gc.SpdnnError):
        gc.reference_bias(1000)
    # file names (reference src/network.cpp:14-19)
    assert gc.weight_file_name("../data", 1024, 0) == "../data/neuron1024/n1024-l1.tsv"
    assert gc.weight_file_name("/d", 65536, 1919) == "/d/neuron65536/n65536-l1920.tsv"
    # HashReorder closed form (reference src/reorder/hash.h:14-22): bijection, reorder(65) = 17 at (64, 1024)
    assert gc.hash_reorder(65, 64, 1024) == 17
    assert sorted(gc.hash_reorder(v, 64, 1024) for v in range(1024)) == list(range(1024))
    with pytest.raises(gc.SpdnnError):
        gc.hash_reorder(1024, 64, 1024)


def _emulate_band_layer(net, l, y_phys, value_of):
    """CPU emulation of the band kernel from the plan arrays: ring selectors, accumulation in
    plan order, output scattered through dst."""
    n = net.neuron
    in_pos, out_at, sel = net.band_plan(l)
    dst = net.layer_dst(l)
    k = sel.shape[1]
    halo = net.layer_plan(l).band_halo
    out = np.zeros_like(y_phys)
    for v in range(n):
        acc = np.zeros(y_phys.shape[0], np.float32)
        # what the ring of a 16-output chunk holds: the chunk's own positions and the halo before it
        top = v // 16 * 16 + 15
        window = [(top - d) % n for d in range(halo + 16)]
        by_slot = {p % 256: p for p in window}
        assert len(by_slot) == halo + 16
        for m in range(k):
            p = by_slot[int(sel[v, m])]
            acc = acc + y_phys[:, p] * value_of(v, m)
        y = acc + np.float32(net.bias)
        out[:, dst[v]] = np.where(y < 0, np.float32(0), np.where(y > 32, np.float32(32), y))
    return out


def test_inspector_band_plan_reproduces_oracle(gc, orc):
    n, L, b = 512, 3, 6
    layers = [orc.gen_layer_csr(11, l, n) for l in range(L)]
    with gc.Network(n, b, L, bias=-0.3) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        for l in range(L):
            p = net.layer_plan(l)
            assert (p.kernel, p.max_row_nnz, p.regular, p.uniform_value, p.exact_products, p.band_halo, p.nnz) == \
                   (gc.KERNEL_BAND, 32, 1, 1, 1, 31, 32 * n)
            in_pos, out_at, sel = net.band_plan(l)
            assert sorted(in_pos.tolist()) == list(range(n)) and sorted(out_at.tolist()) == list(range(n))
            # every output reads exactly the window behind its band position
            rowptr, col, _ = layers[l]
            for v in (0, 1, 31, 32, n - 1):
                want = {(v - d) % n for d in range(32)}
                assert {int(in_pos[i]) for i in col[rowptr[out_at[v]]:rowptr[out_at[v] + 1]]} == want
        assert np.array_equal(net.input_labelling(L), np.arange(n))
        feats = orc.gen_features(11, n, 0, b, 0.1, 0.5)
        y = np.zeros_like(feats)
        y[:, net.input_labelling(0)] = feats
        want = feats
        for l in range(L):
            y = _emulate_band_layer(net, l, y, lambda v, m: np.float32(0.0625))
            want, _ = orc.layer(want, layers[l], -0.3)
            assert np.array_equal(y[:, net.input_labelling(l + 1)], want)


def _emulate_band_pairs(net, l, y_phys, uniform_value):
    """CPU emulation of the band kernel from the pair records it streams: per pair of neighbouring
    band positions one merged list of steps; a step's column is read once and added into the
    accumulators of the outputs whose use bit is set."""
    n = net.neuron
    steps, rec, w = net.band_pairs(l)
    halo = net.layer_plan(l).band_halo
    dst = net.layer_dst(l)
    out = np.zeros_like(y_phys)
    slots = rec[:, 4:].copy().view(np.uint8)
    for u in range(n // 2):
        use = [int(rec[u, 0]) | int(rec[u, 1]) << 32, int(rec[u, 2]) | int(rec[u, 3]) << 32]
        top = (2 * u) // 16 * 16 + 15
        by_slot = {p % 256: p for p in ((top - d) % n for d in range(halo + 16))}
        acc = [np.zeros(y_phys.shape[0], np.float32), np.zeros(y_phys.shape[0], np.float32)]
        for m in range(steps):
            x = y_phys[:, by_slot[int(slots[u, m])]]
            for o in (0, 1):
                if w is not None:
                    acc[o] = acc[o] + x * w[u, m, o]            # 0 where the output does not use the step
                    assert (w[u, m, o] != 0) == bool(use[o] >> m & 1) or w[u, m, o] == 0
                elif use[o] >> m & 1:
                    acc[o] = acc[o] + x * np.float32(uniform_value)
        assert all(use[o] >> steps == 0 for o in (0, 1))
        for o in (0, 1):
            y = acc[o] + np.float32(net.bias)
            out[:, dst[2 * u + o]] = np.where(y < 0, np.float32(0), np.where(y > 32, np.float32(32), y))
    return out


def test_band_pair_records_reproduce_oracle(gc, orc, monkeypatch):
    """The merged step lists of output pairs, for circulant bands (33 steps for 32 entries, 9 for
    8), run chains (32 steps) and general weights, emulated on the CPU against the oracle."""
    monkeypatch.setenv("SPDNN_RUN_CHAINS_MIN_N", "256")
    n, b = 512, 5
    rng = np.random.default_rng(21)
    band8 = orc.gen_layer_csr(4, 1, n, 8)
    layers = [orc.gen_layer_csr(4, 0, n), radix_like_csr(rng, n, 64, "uniform"), band8,
              (band8[0], band8[1], rng.uniform(-0.1, 0.15, size=len(band8[1])).astype(np.float32)),
              radix_like_csr(rng, n, 16, "general")]
    with gc.Network(n, b, len(layers), bias=-0.1) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert [net.band_pairs(l)[0] for l in range(len(layers))] == [33, 32, 9, 9, 32]
        assert [net.band_pairs(l)[1].shape[1] for l in range(len(layers))] == [16] * 5   # one record size
        assert [net.band_pairs(l)[2] is None for l in range(len(layers))] == [True, True, True, False, False]
        feats = orc.gen_features(4, n, 0, b, 0.2, 0.7) * np.float32(1.7)
        y = np.zeros_like(feats)
        y[:, net.input_labelling(0)] = feats
        want = feats
        for l, csr in enumerate(layers):
            y = _emulate_band_pairs(net, l, y, 0.0625)
            want, _ = orc.layer(want, csr, -0.1)
            assert np.array_equal(y[:, net.input_labelling(l + 1)], want), l


def _emulate_band_quads(net, l, y_phys):
    """CPU emulation of the resident band launch from the QUAD form it streams: the four outputs at band positions
    4c .. 4c+3 walk one merged list of steps; a step's column enters every output with the step's weight in that
    output (0 where the output does not use it), rounded multiply then rounded add as the reference does."""
    n = net.neuron
    groups, cols, w = net.band_quads(l)
    assert groups > 0
    dst = net.layer_dst(l)
    out = np.zeros_like(y_phys)
    assert (cols % 64 == 0).all() and (cols // 64 < n).all()
    for c in range(n // 4):
        acc = [np.zeros(y_phys.shape[0], np.float32) for _ in range(4)]
        for g in range(groups):
            for k in range(4):
                x = y_phys[:, int(cols[c, g, k]) // 64]
                for o in range(4):
                    acc[o] = acc[o] + x * w[c, g, k, o]
        for o in range(4):
            y = acc[o] + np.float32(net.bias)
            out[:, dst[4 * c + o]] = np.where(y < 0, np.float32(0), np.where(y > 32, np.float32(32), y))
    return out


def test_band_quad_form_reproduces_oracle(gc, orc, monkeypatch):
    """The merged step lists of output quads that the resident launches of band layers stream (35 steps in 9 groups for
    32 entries per row, 11 in 3 for 8), for circulant bands with one weight and with general weights and for run
    chains, emulated on the CPU against the oracle; a layer wider than 1024 neurons carries no such form."""
    monkeypatch.setenv("SPDNN_RUN_CHAINS_MIN_N", "256")
    n, b = 512, 5
    rng = np.random.default_rng(23)
    band8 = orc.gen_layer_csr(4, 1, n, 8)
    band32 = orc.gen_layer_csr(4, 2, n)
    layers = [orc.gen_layer_csr(4, 0, n), band8,
              (band8[0], band8[1], rng.uniform(-0.1, 0.15, size=len(band8[1])).astype(np.float32)),
              (band32[0], band32[1], np.ldexp(1.0, rng.integers(-6, -3, size=len(band32[1]))).astype(np.float32)),
              radix_like_csr(rng, n, 16, "general")]
    with gc.Network(n, b, len(layers), bias=-0.1) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert [net.layer_plan(l).kernel for l in range(len(layers))] == [gc.KERNEL_BAND] * len(layers)
        assert [net.band_quads(l)[0] for l in range(len(layers))] == [9, 3, 3, 9, 8]
        feats = orc.gen_features(4, n, 0, b, 0.2, 0.7) * np.float32(1.7)
        y = np.zeros_like(feats)
        y[:, net.input_labelling(0)] = feats
        want = feats
        for l, csr in enumerate(layers):
            y = _emulate_band_quads(net, l, y)
            want, _ = orc.layer(want, csr, -0.1)
            assert np.array_equal(y[:, net.input_labelling(l + 1)], want), l
    wide = 2048
    with gc.Network(wide, b, 1, bias=-0.1) as net:
        net.set_layer_csr(0, *orc.gen_layer_csr(4, 0, wide))
        net.inspect()
        assert net.layer_plan(0).kernel == gc.KERNEL_BAND and net.band_quads(0)[0] == 0



@pytest.mark.parametrize("tiled", [1, 0])
def test_inspector_falls_back_to_the_general_classes(gc, orc, tiled, monkeypatch):
    monkeypatch.setenv("SPDNN_TILED", str(tiled))
    general = gc.KERNEL_TILED if tiled else gc.KERNEL_GATHER
    rng = np.random.default_rng(3)
    n = 256
    irregular = random_csr(rng, n, rng.integers(0, 20, size=n), "general")
    # 8 entries per row AND per column, no band and no two outputs with the same inputs:
    # output j reads inputs (4k+1)*j + k (mod n), k = 0..7 (eight affine bijections of Z_n)
    cols = np.sort((np.arange(n)[:, None] * (4 * np.arange(8)[None, :] + 1) + np.arange(8)[None, :]) % n, axis=1)
    assert all(len(set(r)) == 8 for r in cols) and (np.bincount(cols.reshape(-1), minlength=n) == 8).all()
    regular_random = (np.arange(0, 8 * n + 1, 8, dtype=np.int32), cols.reshape(-1).astype(np.int32),
                      np.full(8 * n, 0.0625, np.float32))
    band = orc.gen_layer_csr(2, 0, n, 8)
    with gc.Network(n, 4, 4, bias=0.0) as net:
        net.set_layer_csr(0, *irregular)
        net.set_layer_csr(1, *regular_random)
        net.set_layer_csr(2, *band)
        net.set_layer_csr(3, band[0], band[1], np.linspace(0.1, 0.2, len(band[1])).astype(np.float32))
        net.inspect()
        p = [net.layer_plan(l) for l in range(4)]
        assert [q.kernel for q in p] == [general, general, gc.KERNEL_BAND, gc.KERNEL_BAND]
        assert (p[0].regular, p[0].exact_products) == (0, 0) and p[0].band_halo == -1
        assert (p[1].regular, p[1].uniform_value, p[1].exact_products) == (1, 1, 1)
        assert (p[2].max_row_nnz, p[2].band_halo) == (8, 7)
        assert (p[3].uniform_value, p[3].exact_products) == (0, 0)
        with pytest.raises(gc.SpdnnError) as e:
            net.band_plan(0)
        assert e.value.code == 2
        # a general layer reads its input in natural order; its outputs go where the next layer reads
        assert np.array_equal(net.input_labelling(0), np.arange(n))
        d1 = net.layer_dst(1)      # gather: one slot per neuron; tiled: 1024 slots per tile, -1 where unused
        assert np.array_equal(np.sort(d1[d1 >= 0]), np.arange(n)) and (len(d1) == n or len(d1) == 1024)
        if not tiled:
            assert np.array_equal(d1, net.input_labelling(2))
        assert np.array_equal(net.layer_dst(3), np.arange(n)[net.band_plan(3)[1]])


def test_inspector_block_class(gc, orc):
    """Outputs that read identical input lists are grouped (RadiX-Net style), whatever the
    labelling; the plan lists every output exactly once."""
    rng = np.random.default_rng(5)
    n = 512
    with gc.Network(n, 4, 3, bias=-0.3) as net:
        net.set_layer_csr(0, *hub_block_csr(rng, n, "uniform"))              # one run read by every group
        net.set_layer_csr(1, *hub_block_csr(rng, n, "general"))
        net.set_layer_csr(2, *radix_like_csr(rng, n, 128, "pow2", run=8))   # groups of 8 outputs, 16 inputs
        net.inspect()
        p = [net.layer_plan(l) for l in range(3)]
        assert [q.kernel for q in p] == [gc.KERNEL_BLOCK] * 3
        assert (p[0].max_row_nnz, p[0].uniform_value, p[0].exact_products, p[0].regular) == (32, 1, 1, 0)
        assert (p[1].uniform_value, p[1].exact_products) == (0, 0)
        assert p[2].max_row_nnz == 16
        for l in range(3):
            dst = net.layer_dst(l)
            used = dst[dst >= 0]
            assert sorted(used.tolist()) == list(range(n))
    with gc.Network(n, 4, 1, bias=-0.3, force_kernel=gc.KERNEL_GATHER) as net:
        net.set_layer_csr(0, *radix_like_csr(rng, n, 64, "uniform"))
        net.inspect()
        assert net.layer_plan(0).kernel == gc.KERNEL_GATHER
    # chains of groups: BLOCK below 4096 neurons, walked by the band kernel from there up
    for width, kind, halo in ((512, gc.KERNEL_BLOCK, -1), (4096, gc.KERNEL_BAND, 32)):
        with gc.Network(width, 4, 1, bias=-0.3) as net:
            net.set_layer_csr(0, *radix_like_csr(rng, width, 64, "uniform"))
            net.inspect()
            assert (net.layer_plan(0).kernel, net.layer_plan(0).band_halo) == (kind, halo)


@pytest.mark.parametrize("n", [256, 768, 1024])
def test_inspector_run_chains(gc, orc, n, monkeypatch):
    """RadiX-Net layers - groups of 16 outputs reading two 16-wide input runs, every run read by
    two groups - are laid out as chains and walked by the band kernel with a halo of 32: every
    stride (one long cycle, several cycles, cycles of three and of two groups), hidden behind
    random relabellings."""
    monkeypatch.setenv("SPDNN_RUN_CHAINS_MIN_N", "256")   # the default keeps widths below 4096 on the BLOCK kernel
    rng = np.random.default_rng(n)
    strides = [16, 32, 48, 64, 80, n // 4, n // 2, n - 16]
    if n % 3 == 0:
        strides += [n // 3, 16 * 15]               # 16 cycles of three groups; three cycles of 16
    L, b = len(strides), 5
    layers = [radix_like_csr(rng, n, st, "general" if i % 2 else "uniform") for i, st in enumerate(strides)]
    with gc.Network(n, b, L, bias=-0.3) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        for l in range(L):
            p = net.layer_plan(l)
            assert (p.kernel, p.max_row_nnz, p.regular, p.band_halo) == (gc.KERNEL_BAND, 32, 1, 32), strides[l]
            assert p.block_form == (0 if l % 2 else 1)   # with one exact value the layer keeps its BLOCK form too
            in_pos, out_at, sel = net.band_plan(l)
            assert sorted(in_pos.tolist()) == list(range(n)) and sorted(out_at.tolist()) == list(range(n))
            rowptr, col, _ = layers[l]
            for v in range(n):
                top = v // 16 * 16 + 15
                back = (top - in_pos[col[rowptr[out_at[v]]:rowptr[out_at[v] + 1]]]) % n
                assert back.max() <= 47, (strides[l], v)
        feats = orc.gen_features(11, n, 0, b, 0.1, 0.5)
        y = np.zeros_like(feats)
        y[:, net.input_labelling(0)] = feats
        want = feats
        for l in range(L):
            rowptr, col, val = layers[l]
            _, out_at, _ = net.band_plan(l)
            y = _emulate_band_layer(net, l, y, lambda v, m: val[rowptr[out_at[v]] + m])
            want, _ = orc.layer(want, layers[l], -0.3)
            assert np.array_equal(y[:, net.input_labelling(l + 1)], want), strides[l]


def test_receptive_field_of_every_layer_class(gc, orc, monkeypatch):
    """spdnn_receptive_field (the reference's FuseLayer analysis, src/fuse/fuse.h:13-53) works from the
    inspector's plans: compare with the oracle on the CSR that was handed over, for band, run-chain,
    block and gather layers, through one to four layers."""
    monkeypatch.setenv("SPDNN_RUN_CHAINS_MIN_N", "512")
    rng = np.random.default_rng(21)
    n = 512
    layers = [orc.gen_layer_csr(3, 0, n), radix_like_csr(rng, n, 64), hub_block_csr(rng, n),
              sort_rows(random_csr(rng, n, rng.integers(0, 9, size=n), "general")), orc.gen_layer_csr(3, 1, n)]
    with gc.Network(n, 4, len(layers), bias=-0.3) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        kinds = [net.layer_plan(l).kernel for l in range(len(layers))]
        assert kinds == [gc.KERNEL_BAND, gc.KERNEL_BAND, gc.KERNEL_BLOCK, gc.KERNEL_TILED, gc.KERNEL_BAND]
        assert net.layer_plan(1).band_halo == 32
        for first in range(len(layers)):
            for depth in range(1, len(layers) - first + 1):
                for outs in (np.arange(16), np.array([7]), rng.choice(n, 40, replace=False), np.arange(n)):
                    got = net.receptive_field(first, depth, outs)
                    assert np.array_equal(got, orc.receptive_field(layers[first:first + depth], outs))
        with pytest.raises(gc.SpdnnError):
            net.receptive_field(0, len(layers) + 1, [0])
        with pytest.raises(gc.SpdnnError):
            net.receptive_field(0, 1, [n])
    with gc.Network(n, 4, 1, bias=-0.3, force_kernel=gc.KERNEL_GATHER) as net:
        net.set_layer_csr(0, *layers[3])
        net.inspect()
        assert net.layer_plan(0).kernel == gc.KERNEL_GATHER
        assert np.array_equal(net.receptive_field(0, 1, np.arange(40)), orc.receptive_field(layers[3:4], np.arange(40)))


def test_fusable_pairs_are_found_by_the_inspector(gc, orc):
    """Layers that are bands over one common neuron order write their outputs where the next one reads
    them: the inspector gives them one labelling (dst = identity) and marks the pairs; the receptive
    field of a tile through such a pair is the tile plus a halo, through a pair of the generator's
    layers (a fresh permutation per layer) it is all but the whole row."""
    rng = np.random.default_rng(22)
    n = 1024
    perm = rng.permutation(n)
    flipped = perm[::-1].copy()
    layers = [common_band_csr(rng, n, perm), common_band_csr(rng, n, perm, "pow2"), common_band_csr(rng, n, perm, "pow2"),
              common_band_csr(rng, n, flipped, "pow2"), orc.gen_layer_csr(4, 0, n), orc.gen_layer_csr(4, 1, n)]
    with gc.Network(n, 4, len(layers), bias=-0.3) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        for l in range(4):     # the same places along the band for a neuron as input and as output, neuron 0 first
            in_pos, out_at, _ = net.band_plan(l)
            assert in_pos[0] == 0 and np.array_equal(in_pos[out_at], np.arange(n))
        # layers 0-1 differ in weight mode, 1-2 fuse, 2-3 are bands over opposite orders, 3-4 and 4-5 unrelated
        assert [net.layer_plan(l).fuse_next for l in range(len(layers))] == [0, 1, 0, 0, 0, 0]
        assert np.array_equal(net.layer_dst(0), np.arange(n)) and np.array_equal(net.layer_dst(1), np.arange(n))
        in_pos, out_at, _ = net.band_plan(2)
        tile = out_at[256:256 + 64]                     # 64 consecutive band positions of layer 2
        assert len(net.receptive_field(1, 2, tile)) == 64 + 2 * 31
        assert len(net.receptive_field(1, 1, tile)) == 64 + 31
        in_pos, out_at, _ = net.band_plan(5)
        assert len(net.receptive_field(4, 2, out_at[:64])) > 0.95 * n


def test_radix_layers_of_one_numbering_share_an_order(gc, orc):
    """RadiX-Net layers whose files share a hidden neuron numbering: the inspector lays the layers of
    stride 16 and 32 out in one common order (the cycle of the stride-16 layer), so that neighbours
    among them write where the next one reads and are marked for the fused launch; wider strides and
    layers with a numbering of their own keep their own labelling.  The structure the plans describe
    stays the layer's."""
    rng = np.random.default_rng(31)
    n = 4096
    perm = rng.permutation(n)
    strides = [16, 32, 64, 2048, 16, 32, 32, 16, None, 16]
    layers = [radix_like_csr(rng, n, s, perm=perm) if s else radix_like_csr(rng, n, 16) for s in strides]
    with gc.Network(n, 4, len(layers), bias=-0.3) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        plans = [net.layer_plan(l) for l in range(len(layers))]
        assert [p.kernel for p in plans] == [gc.KERNEL_BAND] * len(layers)
        assert [p.common_order for p in plans] == [1, 2, 0, 0, 1, 2, 2, 1, 0, 1]
        assert [p.fuse_next for p in plans] == [1, 0, 0, 0, 1, 1, 1, 0, 0, 0]
        in0, out0, _ = net.band_plan(0)
        assert np.array_equal(in0[out0], np.arange(n))           # one place per neuron, as input and as output
        for l in (1, 4, 5, 6, 7, 9):
            in_pos, out_at, _ = net.band_plan(l)
            assert np.array_equal(in_pos, in0) and np.array_equal(out_at, out0)
        for l in (0, 4, 5, 6):
            assert np.array_equal(net.layer_dst(l), np.arange(n))
        # the neurons of a 16-wide slot are one block of the hidden numbering
        inv = np.argsort(perm)
        assert all(len(set(inv[out0[16 * t:16 * t + 16]] // 16)) == 1 for t in range(n // 16))
        for l in (0, 1, 5, 8):
            assert np.array_equal(net.receptive_field(l, 1, np.arange(n)), np.arange(n))
            some = np.arange(40, 56)
            assert np.array_equal(net.receptive_field(l, 1, some), orc.receptive_field(layers[l:l + 1], some))
        net.inspect()    # a second call finds the order again and leaves the layers as they are
        assert [net.layer_plan(l).common_order for l in range(len(layers))] == [1, 2, 0, 0, 1, 2, 2, 1, 0, 1]


def test_forced_gather(gc, orc):
    with gc.Network(256, 4, 2, bias=-0.3, force_kernel=gc.KERNEL_GATHER) as net:
        net.synth_layers(0, nnz_per_row=8)
        net.inspect()
        assert [net.layer_plan(l).kernel for l in range(2)] == [gc.KERNEL_GATHER] * 2


def test_tsv_layer_through_the_library(gc, orc, tmp_path):
    """A layer written as a shuffled challenge-format TSV and loaded by the library gives the
    same plan as the same layer handed over as CSR."""
    n = 256
    csr = orc.gen_layer_csr(6, 0, n, 8)
    rowptr, col, val = csr
    lines = ["%d\t%d\t%.9g\n" % (col[e] + 1, j + 1, val[e]) for j in range(n) for e in range(rowptr[j], rowptr[j + 1])]
    np.random.default_rng(0).shuffle(lines)
    p = tmp_path / "n256-l1.tsv"
    p.write_text("".join(lines))
    with gc.Network(n, 4, 1, bias=-0.3) as a, gc.Network(n, 4, 1, bias=-0.3) as b:
        a.load_layer_tsv(0, str(p))
        b.set_layer_csr(0, *csr)
        a.inspect()
        b.inspect()
        for x, y in zip(a.band_plan(0), b.band_plan(0)):
            assert np.array_equal(x, y)
        with pytest.raises(gc.SpdnnError) as e:
            a.load_layer_tsv(0, str(tmp_path / "missing.tsv"))
        assert e.value.code == 3 and "does not exists" in e.value.message
        # an index that does not fit 32 bits is out of range, not the neuron it would wrap round to
        for bad in ("4294967297\t1\t0.5\n", "1\t4294967297\t0.5\n", "-4294967295\t1\t0.5\n", "0\t1\t0.5\n"):
            q = tmp_path / "wrap.tsv"
            q.write_text("".join(lines[:5]) + bad)
            with pytest.raises(gc.SpdnnError) as e:
                a.load_layer_tsv(0, str(q))
            assert e.value.code == 3 and "out of range" in e.value.message
    # the committed fixture layers are plain (non-band) layers of width 64
    with gc.Network(64, 12, 2, bias=-0.3) as net:
        net.load_layer_tsv(0, os.path.join(GOLD, "tiny_n64-l1.tsv"))
        net.load_layer_tsv(1, os.path.join(GOLD, "tiny_n64-l2.tsv"))
        net.inspect()
        assert net.layer_plan(0).nnz == 64 * 8


def test_tsv_directory_loaded_in_parallel(gc, orc, tmp_path):
    """All layers of a data directory (the reference's file names) in one call: same plans as the
    layers handed over one by one; a missing or broken file is reported by name."""
    n, L = 256, 7
    d = tmp_path / ("neuron%d" % n)
    d.mkdir()
    layers = [orc.gen_layer_csr(8, l, n, 8) for l in range(L)]
    rng = np.random.default_rng(1)
    for l, (rowptr, col, val) in enumerate(layers):
        lines = ["%d\t%d\t%.9g\n" % (col[e] + 1, j + 1, val[e]) for j in range(n) for e in range(rowptr[j], rowptr[j + 1])]
        rng.shuffle(lines)
        (d / ("n%d-l%d.tsv" % (n, l + 1))).write_text("".join(lines))
    with gc.Network(n, 4, L, bias=-0.3) as a, gc.Network(n, 4, L, bias=-0.3) as b:
        a.load_layers_tsv(tmp_path)
        for l, csr in enumerate(layers):
            b.set_layer_csr(l, *csr)
        a.inspect()
        b.inspect()
        for l in range(L):
            for x, y in zip(a.band_plan(l), b.band_plan(l)):
                assert np.array_equal(x, y)
            assert np.array_equal(a.layer_dst(l), b.layer_dst(l))
        # a part of the range, then a file that is not there, then one with a bad index
        a.load_layers_tsv(tmp_path, first=2, count=3)
        a.inspect()
        (d / ("n%d-l4.tsv" % n)).unlink()
        with pytest.raises(gc.SpdnnError) as e:
            a.load_layers_tsv(tmp_path)
        assert e.value.code == 3 and "n256-l4.tsv" in e.value.message
        with pytest.raises(gc.SpdnnError) as e:
            a.inspect()                                 # layer 3 stayed unset
        assert e.value.code == 2
        (d / ("n%d-l4.tsv" % n)).write_text("1\t%d\t0.5\n" % (n + 1))
        with pytest.raises(gc.SpdnnError) as e:
            a.load_layers_tsv(tmp_path)
        assert "n256-l4.tsv" in e.value.message
        with pytest.raises(gc.SpdnnError):
            a.load_layers_tsv(tmp_path, first=5, count=4)


def test_features_tsv_parsed_in_parts(gc, orc, tmp_path):
    """A feature file of several MiB (parsed in parts by several threads) against the oracle's
    reader: shuffled lines, rows beyond the batch, values with fractions and exponents; then the
    same file with an entry set twice far apart (the later line must win) and with a triple that
    straddles a line end (accepted, as stream extraction does)."""
    N, B = 512, 1500
    rng = np.random.default_rng(5)
    flat = rng.choice(N * (B + 100), size=400000, replace=False)
    rows, cols = flat // N + 1, flat % N + 1
    vals = np.where(rng.random(len(flat)) < 0.7, 1.0, rng.uniform(0.001, 30.0, len(flat))).astype(np.float32)
    lines = ["%d\t%d\t%s\n" % (r, c, "1" if v == 1.0 else ("%.6e" % v if i % 3 else "%.7f" % v))
             for i, (r, c, v) in enumerate(zip(rows.tolist(), cols.tolist(), vals.tolist()))]
    p = tmp_path / "sparse-images-512.tsv"
    p.write_text("".join(lines))
    assert p.stat().st_size > (4 << 20)
    want, want_kept = orc.read_features_tsv(str(p), N, B)
    got, kept = gc.read_features_tsv(p, N, B)
    assert kept == want_kept == int((rows <= B).sum())
    assert same_floats(got, want)
    # the first entry again at the very end with another value, and a triple broken over two lines
    r0, c0 = int(rows[rows <= B][0]), int(cols[rows <= B][0])
    p.write_text("".join(lines) + "%d\t%d\t7.25\n" % (r0, c0) + "3\t9\n2.5\n")
    want, want_kept = orc.read_features_tsv(str(p), N, B)
    got, kept = gc.read_features_tsv(p, N, B)
    assert got[r0 - 1, c0 - 1] == np.float32(7.25) and got[2, 8] == np.float32(2.5)
    assert kept == want_kept and same_floats(got, want)
    # errors: an index out of range in the middle, a line that is no triple, a missing file
    bad = list(lines)
    bad[len(bad) // 2] = "5\t%d\t1\n" % (N + 1)
    p.write_text("".join(bad))
    with pytest.raises(gc.SpdnnError) as e:
        gc.read_features_tsv(p, N, B)
    assert e.value.code == 3 and "out of range" in e.value.message
    bad[len(bad) // 2] = "5\tx\t1\n"
    p.write_text("".join(bad))
    with pytest.raises(gc.SpdnnError) as e:
        gc.read_features_tsv(p, N, B)
    assert "malformed" in e.value.message
    with pytest.raises(gc.SpdnnError):
        gc.read_features_tsv(tmp_path / "nothing.tsv", N, B)


def _write_weights_bin(path, layers):
    """Packed weight file in the layout readweights of the reference's library benchmark reads
    (benchmark/cusparse/cusparse.cu:340-347): per layer row[], col[], val[], 1-based, row = output."""
    rng = np.random.default_rng(3)
    with open(path, "wb") as f:
        for rowptr, col, val in layers:
            row = np.repeat(np.arange(len(rowptr) - 1, dtype=np.int32), np.diff(rowptr))
            perm = rng.permutation(len(col))
            (row[perm] + 1).astype("<i4").tofile(f)
            (col[perm] + 1).astype("<i4").tofile(f)
            val[perm].astype("<f4").tofile(f)


def test_packed_binary_layers_through_the_library(gc, orc, tmp_path):
    n = 256
    layers = [orc.gen_layer_csr(8, l, n, 32) for l in range(3)]
    p = tmp_path / "neuron256.bin"
    _write_weights_bin(p, layers)
    for l in range(3):   # the oracle's reader gives the layers back (rows sorted by input index)
        rowptr, col, val = orc.read_weights_bin(str(p), n, l)
        srt = [np.sort(col[rowptr[j]:rowptr[j + 1]]) for j in range(n)]
        assert np.array_equal(rowptr, layers[l][0]) and np.array_equal(np.concatenate(srt), layers[l][1])
        assert np.all(val == np.float32(0.0625))
    with gc.Network(n, 4, 3, bias=-0.3) as a, gc.Network(n, 4, 3, bias=-0.3) as b:
        a.load_layers_bin(str(p))
        for l in range(3):
            b.set_layer_csr(l, *layers[l])
        a.inspect()
        b.inspect()
        for l in range(3):
            assert a.layer_plan(l).kernel == gc.KERNEL_BAND
            for x, y in zip(a.band_plan(l), b.band_plan(l)):
                assert np.array_equal(x, y)
            assert np.array_equal(a.layer_dst(l), b.layer_dst(l))
        # a single record out of the middle, and the error paths
        a.load_layers_bin(str(p), first=1, count=1)
        with pytest.raises(gc.SpdnnError) as e:
            a.load_layers_bin(str(tmp_path / "missing.bin"))
        assert e.value.code == 3
        with pytest.raises(gc.SpdnnError) as e:
            a.load_layers_bin(str(p), first=2, count=2)
        assert e.value.code == 1
    with gc.Network(n, 4, 4, bias=-0.3) as c:
        with pytest.raises(gc.SpdnnError) as e:     # the file holds three records only
            c.load_layers_bin(str(p))
        assert e.value.code == 3 and "short read" in e.value.message


def test_argument_and_state_errors(gc, orc):
    E_ARG, E_STATE = 1, 2
    with pytest.raises(gc.SpdnnError) as e:
        gc.Network(0, 4, 1, bias=0.0)
    assert e.value.code == E_ARG
    with pytest.raises(gc.SpdnnError):
        gc.Network(64, 0, 1, bias=0.0)
    with pytest.raises(gc.SpdnnError):
        gc.Network(64, 4, 1, bias=float("nan"))
    with pytest.raises(gc.SpdnnError):
        gc.Network(64, 4, 1, bias=-0.3, clamp=1e31)
    n = 64
    good = sort_rows(random_csr(np.random.default_rng(1), n, 4, "uniform"))
    with gc.Network(n, 4, 2, bias=-0.1) as net:
        with pytest.raises(gc.SpdnnError) as e:
            net.set_layer_csr(2, *good)
        assert e.value.code == E_ARG
        bad_col = good[1].copy()
        bad_col[5] = n
        with pytest.raises(gc.SpdnnError) as e:
            net.set_layer_csr(0, good[0], bad_col, good[2])
        assert e.value.code == E_ARG and "out of range" in e.value.message
        bad_val = good[2].copy()
        bad_val[0] = np.inf
        with pytest.raises(gc.SpdnnError) as e:
            net.set_layer_csr(0, good[0], good[1], bad_val)
        assert "non-finite" in e.value.message
        bad_val[0] = 4.0e6                          # beyond 2^21
        with pytest.raises(gc.SpdnnError) as e:
            net.set_layer_csr(0, good[0], good[1], bad_val)
        assert "2^21" in e.value.message
        bad_ptr = good[0].copy()
        bad_ptr[3] = bad_ptr[2] - 1
        with pytest.raises(gc.SpdnnError):
            net.set_layer_csr(0, bad_ptr, good[1], good[2])
        for slots in (1, -2, 65):                   # the plan window is 0 or 2..64 slots
            with pytest.raises(gc.SpdnnError) as e:
                net.set_plan_window(slots)
            assert e.value.code == E_ARG
        net.set_plan_window(2)
        net.set_plan_window(0)
        with pytest.raises(gc.SpdnnError) as e:
            net.plan_memory()                       # nothing uploaded
        assert e.value.code == E_STATE
        net.set_layer_csr(0, *good)
        with pytest.raises(gc.SpdnnError) as e:
            net.inspect()                           # layer 1 missing
        assert e.value.code == E_STATE
        with pytest.raises(gc.SpdnnError) as e:
            net.run()                               # nothing inspected, no features
        assert e.value.code == E_STATE
        with pytest.raises(gc.SpdnnError) as e:
            net.layer_plan(1)
        assert e.value.code == E_STATE
        with pytest.raises(gc.SpdnnError) as e:
            net.band_quads(1)                       # no such layer yet
        assert e.value.code == E_STATE
        with pytest.raises(gc.SpdnnError) as e:
            net.band_quads(7)
        assert e.value.code == E_ARG
        with pytest.raises(gc.SpdnnError) as e:     # features need the inspected network
            net.set_features_dense(np.zeros((4, n), np.float32))
        assert e.value.code == E_STATE
        net.set_layer_csr(1, *good)
        net.inspect()
        with pytest.raises(gc.SpdnnError) as e:
            net.run()                               # still no features
        assert e.value.code == E_STATE
        net.set_layer_csr(1, *good)                 # a layer changed: inspect again before anything else
        with pytest.raises(gc.SpdnnError) as e:
            net.synth_features(0, 4)
        assert e.value.code == E_STATE


def test_replacing_a_layer(gc, orc):
    n = 256
    with gc.Network(n, 4, 1, bias=-0.3) as net:
        net.set_layer_csr(0, *orc.gen_layer_csr(0, 0, n, 8))
        net.set_layer_csr(0, *orc.gen_layer_csr(1, 0, n, 8))     # replaces the first hand-over
        net.inspect()
        other = gc.Network(n, 4, 1, bias=-0.3)
        other.set_layer_csr(0, *orc.gen_layer_csr(1, 0, n, 8))
        other.inspect()
        assert np.array_equal(net.band_plan(0)[0], other.band_plan(0)[0])
        other.close()


def test_driver_usage_paths(gc):
    exe = os.path.join(ROOT, "graphchallenge21_amd", "spdnn_network")
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 0 and "Usage: exe neuron batch layer" in r.stdout      # reference network.cpp:58-61
    r = subprocess.run([exe, "1000", "10", "2"], capture_output=True, text=True)
    assert r.returncode == 2 and "neuron must be one of" in r.stderr


def test_allocation_failure_comes_back_as_a_status(gc):
    """No exception crosses the C ABI and nothing calls std::terminate: with the address space capped,
    a network of 2^28 layers (tens of GB of host bookkeeping) is refused with SPDNN_E_NOMEM and the
    process lives on."""
    import sys
    code = (
        "import resource, sys\n"
        "sys.path.insert(0, %r)\n"
        "import graphchallenge21_amd as gc\n"
        "gc.load_library()\n"
        "resource.setrlimit(resource.RLIMIT_AS, (6 << 30, 6 << 30))\n"
        "try:\n"
        "    gc.Network(1024, 64, 1 << 28, bias=-0.3)\n"
        "    print('created')\n"
        "except gc.SpdnnError as e:\n"
        "    print('status', e.code)\n"
        "with gc.Network(256, 4, 1, bias=-0.3) as net:\n"
        "    print('alive', net.layers)\n" % ROOT)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr[-2000:]
    assert "status 5" in out.stdout and "alive 1" in out.stdout, out.stdout + out.stderr[-500:]
