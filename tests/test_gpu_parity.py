"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle.

Bar: active-row sets (categories) identical after every layer; fp32 activations bit-identical
(the requirement is 1e-5 relative / 1e-6 absolute; accumulating in the reference's order makes
equality attainable, so equality is what is asserted).
"""
import numpy as np
import pytest

from helpers import random_csr, same_floats, sort_rows
from helpers import common_band_csr, hub_block_csr, radix_like_csr

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-5, 1e-6  # the stated tolerance; the tests assert the stricter bit equality


def _layer_by_layer(gc, orc, net, layers, feats, prune):
    """Runs one layer at a time and checks categories and activations after each."""
    B = feats.shape[0]
    ref = orc.infer(feats, layers, net.bias, prune=False, keep=set(range(len(layers))))
    rows = np.arange(B, dtype=np.int32)
    for l in range(len(layers)):
        print("  layer", l, flush=True)
        r = net.run(prune=prune, first_layer=l, n_layers=1, collect_counts=True)
        want_ids = ref["active_ids"][l]
        got_ids = net.categories()
        assert np.array_equal(got_ids, want_ids), "categories differ after layer %d" % l
        assert r.active_rows == len(want_ids)
        assert net.active_count(l) == len(want_ids)
        got = net.activations(rows)
        want = ref["kept"][l][1]
        assert same_floats(got, want), "activations differ after layer %d: max |d| = %g" % (
            l, float(np.abs(got - want).max()))
        assert np.allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("dmax", [0.25, 0.50])
@pytest.mark.parametrize("prune", [True, False])
def test_band_layer_by_layer(gc, orc, prune, dmax):
    N, L, B = 1024, 8, 600
    print("band N=%d L=%d B=%d prune=%s dmax=%g" % (N, L, B, prune, dmax), flush=True)
    layers = [orc.gen_layer_csr(0, l, N) for l in range(L)]
    feats = orc.gen_features(0, N, 0, B, 0.10, dmax)
    with gc.Network(N, B, L) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert all(net.layer_plan(l).kernel == gc.KERNEL_BAND for l in range(L))
        net.set_features_dense(feats)
        _layer_by_layer(gc, orc, net, layers, feats, prune)


def test_device_features_match_host(gc, orc):
    N, L, B = 1024, 2, 700
    print("synth features N=%d B=%d" % (N, B), flush=True)
    with gc.Network(N, B, L) as net:
        net.synth_layers(3)
        net.inspect()
        net.synth_features(7, B, 0.10, 0.25)
        got = net.activations(np.arange(B, dtype=np.int32))
        want = orc.gen_features(7, N, 0, B, 0.10, 0.25)
        assert np.array_equal(got, want)
        assert np.array_equal(net.categories(), np.arange(B))


@pytest.mark.parametrize("prune", [True, False])
def test_full_chain_cfg0_shape(gc, orc, prune):
    """N=1024, 120 layers, B=6000, bias -0.3: the reference's own CPU-runnable case."""
    N, L, B = 1024, 120, 6000
    print("cfg0 chain prune=%s" % prune, flush=True)
    layers = [orc.gen_layer_csr(0, l, N) for l in range(L)]
    feats = orc.gen_features(0, N, 0, B)
    ref = orc.infer(feats, layers[:12], -0.3, prune=True)   # every row is dead long before layer 12
    assert len(ref["active_ids"][-1]) == 0
    with gc.Network(N, B, L) as net:
        net.synth_layers(0)
        net.inspect()
        net.synth_features(0, B)
        r = net.run(prune=prune, collect_counts=True)
        counts = [net.active_count(l) for l in range(L)]
        assert counts[:12] == [len(a) for a in ref["active_ids"]]
        assert counts[12:] == [0] * (L - 12)
        assert r.active_rows == 0 and len(net.categories()) == 0
        if prune:
            assert r.layers_run < L and r.compactions >= 1
        else:
            assert r.layers_run == L
        # layer by layer at the real batch: the id set and every row's activations after each layer, until
        # everything has died (counts alone would not tell which rows survive)
        ref_u = orc.infer(feats, layers[:12], -0.3, prune=False, keep=set(range(12)))
        rows = np.arange(B, dtype=np.int32)
        checked = 0
        for l in range(12):
            net.run(prune=prune, first_layer=l, n_layers=1, collect_counts=True)
            assert np.array_equal(net.categories(), ref["active_ids"][l]), "layer %d" % l
            assert same_floats(net.activations(rows), ref_u["kept"][l][1]), "layer %d" % l
            checked += 1
            if len(ref["active_ids"][l]) == 0:
                break
        assert checked >= 3 and len(ref["active_ids"][0]) > 1000


def test_survivor_chain_with_compaction(gc, orc):
    """Rows with density up to 0.5 survive and saturate: late-layer pruning and repacks."""
    N, L, B = 1024, 24, 3000
    print("survivor chain", flush=True)
    layers = [orc.gen_layer_csr(5, l, N) for l in range(L)]
    feats = orc.gen_features(5, N, 0, B, 0.10, 0.50)
    ref = orc.infer(feats, layers, -0.3, prune=True)
    assert 0 < len(ref["categories"]) < B
    with gc.Network(N, B, L) as net:
        net.synth_layers(5)
        net.inspect()
        net.set_features_dense(feats)
        for prune in (True, False):
            r = net.run(prune=prune, collect_counts=True)
            assert [net.active_count(l) for l in range(L)] == [len(a) for a in ref["active_ids"]]
            cats = net.categories()
            assert np.array_equal(cats, ref["categories"])
            got = net.activations(cats)
            assert same_floats(got, ref["y"])
            if prune:
                assert r.compactions >= 1
            # pruned rows read back as zero rows
            dead = np.setdiff1d(np.arange(B), cats)[:50].astype(np.int32)
            assert not net.activations(dead).any()


@pytest.mark.parametrize("tiled,rowtile", [(1, 1), (1, 0), (0, 1)])
@pytest.mark.parametrize("values", ["uniform", "pow2", "general"])
def test_gather_kernel_random_sparsity(gc, orc, values, tiled, rowtile, monkeypatch):
    """Irregular rows (0..40 entries), unsorted columns: the general classes - the TILED class in its two forms
    (rows of a workgroup staged in LDS and whole outputs per thread; tiles of outputs with their input columns
    staged in LDS panel by panel) and the plain gather."""
    monkeypatch.setenv("SPDNN_TILED", str(tiled))
    monkeypatch.setenv("SPDNN_ROWTILE", str(rowtile))
    N, L, B = 512, 3, 300
    print("general class tiled=%d rowtile=%d values=%s" % (tiled, rowtile, values), flush=True)
    rng = np.random.default_rng(11)
    layers = [random_csr(rng, N, rng.integers(0, 41, size=N), values) for _ in range(L)]
    feats = rng.uniform(0, 4, size=(B, N)).astype(np.float32) * (rng.random((B, N)) < 0.3)
    feats = feats.astype(np.float32)
    with gc.Network(N, B, L, bias=-0.05) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert all(net.layer_plan(l).kernel == (gc.KERNEL_TILED if tiled else gc.KERNEL_GATHER) for l in range(L))
        net.set_features_dense(feats)
        _layer_by_layer(gc, orc, net, [sort_rows(c) for c in layers], feats, prune=True)


@pytest.mark.parametrize("rowtile", [1, 0])
@pytest.mark.parametrize("min_rows", [0, 8192])
@pytest.mark.parametrize("N", [1024, 2048])
def test_tiled_layers_carry_their_gather_form(gc, orc, N, min_rows, rowtile, monkeypatch):
    """A TILED layer of 1024 neurons or more also holds its GATHER form, and launches below 8192 rows use it (a tile's
    workgroup takes 64 rows x 1024 outputs to itself: too few workgroups on small batches).  Either way the results
    are the oracle's; a run that starts above the threshold and is compacted below it switches form on the way."""
    monkeypatch.setenv("SPDNN_TILED_MIN_ROWS", str(min_rows))
    monkeypatch.setenv("SPDNN_ROWTILE", str(rowtile))     # above the threshold: whole outputs per thread, or the tiles
    L, B = 9, 9000
    print("tiled / gather form N=%d min_rows=%d" % (N, min_rows), flush=True)
    rng = np.random.default_rng(N + min_rows)
    base = [random_csr(rng, N, rng.integers(1, 25, size=N), "general") for _ in range(5)]
    layers = [base[l] if l < 5 else base[2 + l % 3] for l in range(L)]
    dens = np.where(rng.random(B) < 0.25, 0.9, 0.02).astype(np.float32)
    feats = ((rng.random((B, N), dtype=np.float32) < dens[:, None]) * rng.uniform(0.5, 2.0, size=(B, N))).astype(np.float32)
    ref = orc.infer(feats, [sort_rows(c) for c in layers], -0.15, prune=True, keep=set(range(L)))
    want_counts = [len(a) for a in ref["active_ids"]]
    assert 0 < want_counts[4] < 0.5 * B and want_counts[-1] == 0    # (the rows left after layer 4 die in layer 5)
    with gc.Network(N, B, L, bias=-0.15) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert all(net.layer_plan(l).kernel == gc.KERNEL_TILED and net.layer_plan(l).block_form == 2 for l in range(L))
        net.set_features_dense(feats)
        for prune in (True, False):
            r = net.run(prune=prune, collect_counts=True)
            assert (r.compactions >= 1) == prune    # (compacted below 8192 rows on the way)
            assert [net.active_count(l) for l in range(L)] == want_counts
            assert len(net.categories()) == 0
        for l in range(5):
            net.run(prune=True, first_layer=0, n_layers=l + 1)
            gid, y = ref["kept"][l]
            assert np.array_equal(net.categories(), ref["active_ids"][l])
            assert same_floats(net.activations(gid), y)
        net.run(prune=True, first_layer=0, n_layers=3)
        net.run(prune=True, first_layer=3, n_layers=2)     # continued after the compaction
        assert np.array_equal(net.categories(), ref["active_ids"][4])
        assert same_floats(net.activations(ref["kept"][4][0]), ref["kept"][4][1])


@pytest.mark.parametrize("values", ["pow2", "general", "uniform", "uniform-fma"])
@pytest.mark.parametrize("K", [32, 16, 8])
def test_band_kernel_weight_modes(gc, orc, values, K, monkeypatch):
    """Band structure with per-entry weights: exact products (fma) and general (mul then add); with one
    power-of-two weight: inputs added and the sum scaled once, or (switched back) a multiply-add per input."""
    N, L, B = 1024, 3, 260
    print("band weights=%s K=%d" % (values, K), flush=True)
    if values == "uniform-fma":
        monkeypatch.setenv("SPDNN_BAND_SUM_THEN_SCALE", "0")
    rng = np.random.default_rng(K)
    layers = []
    for l in range(L):
        rowptr, col, val = orc.gen_layer_csr(21, l, N, K, 0.0625)
        if values == "pow2":
            val = (np.ldexp(1.0, rng.integers(-5, -1, size=len(val))) * rng.choice([-1.0, 1.0], size=len(val))).astype(np.float32)
        elif values == "general":
            val = rng.uniform(-0.1, 0.2, size=len(val)).astype(np.float32)
        layers.append((rowptr, col, val))
    feats = rng.uniform(0, 2, size=(B, N)).astype(np.float32)
    with gc.Network(N, B, L, bias=-0.1) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert all(net.layer_plan(l).kernel == gc.KERNEL_BAND for l in range(L))
        net.set_features_dense(feats)
        _layer_by_layer(gc, orc, net, layers, feats, prune=True)


@pytest.mark.parametrize("add_only", [1, 0])
@pytest.mark.parametrize("structure", ["circulant", "run-chains"])
@pytest.mark.parametrize("w", [0.0625, -0.5, 2.0 ** -24, 2.0 ** 21, 0.0])
def test_one_power_of_two_weight_sums_then_scales(gc, orc, w, structure, add_only, monkeypatch):
    """A layer whose entries all carry the same weight +-2^e is walked by adding the inputs and scaling the
    sum once.  That equals the reference's multiply-then-add chain bit for bit only because scaling by a
    power of two commutes with rounding: features of both signs over the whole accepted range (2^-100 ..
    2^100, with cancellations down to the last bit), the smallest and largest accepted weights."""
    from helpers import radix_like_csr
    N, L, B = 1024, 3, 300
    print("sum then scale w=%g %s add_only=%d" % (w, structure, add_only), flush=True)
    monkeypatch.setenv("SPDNN_BAND_SUM_THEN_SCALE", str(add_only))   # 0: the same layers with a multiply-add per input
    rng = np.random.default_rng(3)
    if structure == "run-chains":
        monkeypatch.setenv("SPDNN_RUN_CHAINS_MIN_N", "256")
        monkeypatch.setenv("SPDNN_BLOCK_FORM_MAX_ELEMS", "0")
        layers = []
        for l in range(L):
            rp, c, v = radix_like_csr(rng, N, 16 << l, "uniform")
            layers.append((rp, c, np.full(len(v), w, np.float32)))
    else:
        layers = [orc.gen_layer_csr(21, l, N, 32, w) for l in range(L)]
    mag = np.ldexp(rng.uniform(1.0, 2.0, size=(B, N)), rng.integers(-100, 100, size=(B, N)))
    # neighbours that cancel but for the last bits, and rows of moderate values that reach the later layers
    feats = (mag * rng.choice([-1.0, 1.0], size=(B, N)) * (rng.random((B, N)) < 0.7)).astype(np.float32)
    feats[:, 1::2] = np.where(rng.random((B, N // 2)) < 0.5, -np.nextafter(feats[:, 0::2], np.float32(0)), feats[:, 1::2])
    feats[B // 2:] = (rng.uniform(0, 8, size=(B - B // 2, N)) * (rng.random((B - B // 2, N)) < 0.6)).astype(np.float32)
    with gc.Network(N, B, L, bias=-0.1) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert all(net.layer_plan(l).kernel == gc.KERNEL_BAND and net.layer_plan(l).uniform_value for l in range(L))
        net.set_features_dense(feats)
        _layer_by_layer(gc, orc, net, layers, feats, prune=False)


def test_forced_gather_equals_band(gc, orc):
    N, L, B = 1024, 5, 400
    print("forced gather", flush=True)
    layers = [orc.gen_layer_csr(2, l, N) for l in range(L)]
    feats = orc.gen_features(2, N, 0, B, 0.10, 0.5)
    with gc.Network(N, B, L, force_kernel=gc.KERNEL_GATHER) as net:
        net.synth_layers(2)
        net.inspect()
        assert all(net.layer_plan(l).kernel == gc.KERNEL_GATHER for l in range(L))
        net.set_features_dense(feats)
        _layer_by_layer(gc, orc, net, layers, feats, prune=True)


@pytest.mark.parametrize("rl", [1, 2])
def test_other_row_block_sizes(gc, orc, rl, monkeypatch):
    """Row blocks of 64 and 128 rows (the default is 256)."""
    from helpers import hub_block_csr, radix_like_csr
    monkeypatch.setenv("SPDNN_ROWS_PER_LANE", str(rl))
    monkeypatch.setenv("SPDNN_RUN_CHAINS_MIN_N", "256")
    N, L, B = 1024, 4, 333
    print("rows per lane", rl, flush=True)
    layers = [orc.gen_layer_csr(9, l, N) for l in range(L)]
    feats = orc.gen_features(9, N, 0, B, 0.10, 0.5)
    with gc.Network(N, B, L) as net:
        net.synth_layers(9)
        net.inspect()
        net.set_features_dense(feats)
        _layer_by_layer(gc, orc, net, layers, feats, prune=True)
    # the other layer classes at this block size: run chains (one cycle, cycles of two), BLOCK, GATHER
    rng = np.random.default_rng(rl)
    layers = [radix_like_csr(rng, N, 16, "general"), radix_like_csr(rng, N, 512, "uniform"),
              hub_block_csr(rng, N, "pow2"), sort_rows(random_csr(rng, N, rng.integers(1, 20, size=N), "general"))]
    with gc.Network(N, B, 4, bias=-0.2) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert [net.layer_plan(l).kernel for l in range(4)] == [gc.KERNEL_BAND, gc.KERNEL_BAND, gc.KERNEL_BLOCK, gc.KERNEL_TILED]
        net.set_features_dense(feats)
        _layer_by_layer(gc, orc, net, layers, feats, prune=True)


@pytest.mark.parametrize("window", [2, 3])
def test_streamed_plans(gc, orc, window, monkeypatch):
    """Plans streamed through a window of device slots: same results as the oracle (and as resident
    plans), in one run, in continued runs and when run again from the start."""
    from helpers import hub_block_csr, radix_like_csr
    monkeypatch.setenv("SPDNN_RUN_CHAINS_MIN_N", "256")
    N, B = 1024, 700
    rng = np.random.default_rng(40 + window)
    layers = [orc.gen_layer_csr(3, 0, N), radix_like_csr(rng, N, 16, "general"), orc.gen_layer_csr(3, 2, N),
              hub_block_csr(rng, N, "pow2"), orc.gen_layer_csr(3, 4, N),
              sort_rows(random_csr(rng, N, rng.integers(1, 20, size=N), "general")),
              radix_like_csr(rng, N, 512, "uniform"), orc.gen_layer_csr(3, 7, N), orc.gen_layer_csr(3, 8, N)]
    L = len(layers)
    feats = orc.gen_features(3, N, 0, B, 0.10, 0.6)
    rows = np.arange(B, dtype=np.int32)
    for prune in (False, True):
        print("window", window, "prune", prune, flush=True)
        ref = orc.infer(feats, layers, -0.2, prune=False, keep={L - 1})
        with gc.Network(N, B, L, bias=-0.2) as net:
            net.set_plan_window(window)
            for l, csr in enumerate(layers):
                net.set_layer_csr(l, *csr)
            net.inspect()
            kernels = {net.layer_plan(l).kernel for l in range(L)}
            assert kernels == {gc.KERNEL_BAND, gc.KERNEL_BLOCK, gc.KERNEL_TILED}
            net.set_features_dense(feats)
            w, dev_bytes, pinned = net.plan_memory()
            assert w == window and pinned > 0 and dev_bytes > 0   # (window slots of the largest plan's size; all plans pinned)
            with pytest.raises(gc.SpdnnError):
                net.set_plan_window(0)       # too late: the plans are uploaded
            for attempt in range(2):         # the second run starts with the slots as the first left them
                r = net.run(prune=prune, collect_counts=True)
                assert np.array_equal(net.categories(), ref["active_ids"][L - 1])
                assert same_floats(net.activations(rows), ref["kept"][L - 1][1])
                for l in range(L):
                    assert net.active_count(l) == len(ref["active_ids"][l])
            _layer_by_layer(gc, orc, net, layers, feats, prune=prune)
            # three layers, then the rest
            net.run(prune=prune, first_layer=0, n_layers=3)
            net.run(prune=prune, first_layer=3)
            assert np.array_equal(net.categories(), ref["active_ids"][L - 1])
            assert same_floats(net.activations(rows), ref["kept"][L - 1][1])
    # a window as long as the network leaves the plans resident
    with gc.Network(N, B, 2, bias=-0.2) as net:
        net.set_plan_window(2)
        net.synth_layers(3)
        net.inspect()
        net.synth_features(3, B)
        assert net.plan_memory()[0] == 0 and net.plan_memory()[2] == 0


def test_wider_layers(gc, orc):
    """N=4096 and N=16384 at a few layers, rows sampled."""
    for N, bias in ((4096, -0.35), (16384, -0.4)):
        L, B = 4, 520
        print("wide N=%d" % N, flush=True)
        layers = [orc.gen_layer_csr(1, l, N) for l in range(L)]
        feats = orc.gen_features(1, N, 0, B, 0.10, 0.5)
        with gc.Network(N, B, L) as net:
            assert net.bias == pytest.approx(bias)
            net.synth_layers(1)
            net.inspect()
            net.synth_features(1, B, 0.10, 0.5)
            _layer_by_layer(gc, orc, net, layers, feats, prune=True)


def test_committed_tsv_fixtures(gc, orc):
    """Weights and features loaded from the challenge-format TSV fixtures by the library's own
    loaders; expected values from tests/golden/tiny_expected.json (confirmed by the reference's
    CPU comparators when the fixture was generated)."""
    import json
    import os
    gold = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
    exp = json.load(open(os.path.join(gold, "tiny_expected.json")))
    N, B = 64, 12
    print("tsv fixtures", flush=True)
    for bias in (0.0, -1.0, -0.3):
        e = exp["bias_%g" % bias]
        with gc.Network(N, B, 2, bias=bias) as net:
            net.load_layer_tsv(0, os.path.join(gold, "tiny_n64-l1.tsv"))
            net.load_layer_tsv(1, os.path.join(gold, "tiny_n64-l2.tsv"))
            net.inspect()
            net.load_features_tsv(os.path.join(gold, "tiny_features-64.tsv"), B)
            rows = np.arange(B, dtype=np.int32)
            for l, key in ((0, "y_layer1_hex"), (1, "y_layer2_hex")):
                net.run(prune=True, first_layer=l, n_layers=1)
                assert net.categories().tolist() == e["active_ids"][l]
                want = np.frombuffer(bytes.fromhex(e[key]), dtype="<f4").reshape(B, N)
                assert same_floats(net.activations(rows), want)


def test_positive_bias_and_error_paths(gc, orc):
    """bias > 0: dead rows come back to life, so pruning is refused and the unpruned run must
    still be exact (padding rows must never be reported)."""
    N, L, B = 256, 3, 70
    print("positive bias", flush=True)
    layers = [orc.gen_layer_csr(8, l, N, 8, -0.0625) for l in range(L)]
    feats = orc.gen_features(8, N, 0, B, 0.0, 0.3)
    ref = orc.infer(feats, layers, 0.25, prune=False)
    with gc.Network(N, B, L, bias=0.25) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        with pytest.raises(gc.SpdnnError) as e:
            net.set_features_dense(np.full((B + 1, N), 1.0, np.float32))     # more rows than max_batch
        assert e.value.code == 1
        bad = feats.copy()
        bad[5, 7] = np.nan
        with pytest.raises(gc.SpdnnError) as e:
            net.set_features_dense(bad)
        assert e.value.code == 1 and "NaN" in e.value.message
        bad[5, 7] = 1e31                                                     # beyond 2^100
        with pytest.raises(gc.SpdnnError) as e:
            net.set_features_dense(bad)
        assert e.value.code == 1 and "2^100" in e.value.message
        net.set_features_dense(feats)
        with pytest.raises(gc.SpdnnError) as e:
            net.run(prune=True)
        assert e.value.code == 6
        r = net.run(prune=False, collect_counts=True)
        assert np.array_equal(net.categories(), ref["categories"]) and r.active_rows == len(ref["categories"])
        assert same_floats(net.activations(np.arange(B, dtype=np.int32)), ref["y"])


def test_full_batch_properties_cfg1(gc, orc):
    """N=1024, 120 layers, batch 60000 (the first full-GPU configuration), survivor densities so
    that the late layers carry rows: size-independent properties plus an oracle sample."""
    N, L, B = 1024, 120, 60000
    print("cfg1 full batch", flush=True)
    with gc.Network(N, B, L) as net:
        net.synth_layers(0)
        net.inspect()
        net.synth_features(0, B, 0.10, 0.50)
        rp = net.run(prune=True, collect_counts=True)
        counts_p = [net.active_count(l) for l in range(L)]
        cats_p = net.categories()
        sample = np.concatenate([cats_p[:40], cats_p[-40:]]).astype(np.int32)
        y_p = net.activations(sample)
        ru = net.run(prune=False, collect_counts=True)
        counts_u = [net.active_count(l) for l in range(L)]
        cats_u = net.categories()
        y_u = net.activations(sample)
    assert counts_p == counts_u and counts_p == sorted(counts_p, reverse=True)
    assert 0 < counts_p[-1] < B and rp.compactions >= 1 and ru.compactions == 0
    assert np.array_equal(cats_p, cats_u) and np.array_equal(cats_p, np.sort(cats_p))
    assert same_floats(y_p, y_u)
    # oracle on a row sample: rows are independent, so the sample's survivors must be exactly
    # the categories that fall inside the sample
    S = 1500
    layers = [orc.gen_layer_csr(0, l, N) for l in range(L)]
    ref = orc.infer(orc.gen_features(0, N, 0, S, 0.10, 0.50), layers, -0.3, prune=True)
    assert np.array_equal(cats_p[cats_p < S], ref["categories"])
    k = int((sample < S).sum())
    if k:
        pos = np.searchsorted(ref["gid"], sample[:k])
        assert same_floats(y_p[:k], ref["y"][pos])


PERSIST_MODES = {   # how the units of a persistent launch are queued and handed over (environment, read at creation);
                    # light = the writer leaves the write-back of its XCD's L2 out
    "default": {},
    "one-queue": {"SPDNN_PERSIST_XCD": "0"},
    "xcd-queues": {"SPDNN_PERSIST_XCD": "1", "SPDNN_PERSIST_LIGHT_SYNC": "0"},
    "xcd-queues-light": {"SPDNN_PERSIST_XCD": "1", "SPDNN_PERSIST_LIGHT_SYNC": "1"},
}


@pytest.mark.parametrize("mode", sorted(PERSIST_MODES))
@pytest.mark.parametrize("prune", [True, False])
@pytest.mark.parametrize("fuse", [4, 16])
def test_persistent_launches(gc, orc, fuse, prune, mode, monkeypatch):
    """Several band layers per launch with a dependency per row block between the layers must give what the
    layer-by-layer launches give: counts, categories and activations - with one unit queue or one per XCD,
    with device-scope fences or the hand-over inside one XCD's L2."""
    for k, v in PERSIST_MODES[mode].items():
        monkeypatch.setenv(k, v)
    monkeypatch.setenv("SPDNN_BAND_RESIDENT", "0")   # (layers this narrow would share resident launches instead)
    N, L, B = 1024, 24, 3000
    print("persistent launches fuse=%d prune=%s %s" % (fuse, prune, mode), flush=True)
    layers = [orc.gen_layer_csr(5, l, N) for l in range(L)]
    feats = orc.gen_features(5, N, 0, B, 0.10, 0.50)
    ref = orc.infer(feats, layers, -0.3, prune=True)
    with gc.Network(N, B, L) as net:
        net.synth_layers(5)
        net.inspect()
        net.set_features_dense(feats)
        r = net.run(prune=prune, collect_counts=True, fuse_layers=fuse)
        assert r.layers_run == L
        assert r.persistent_launches >= L // fuse and r.persistent_fallbacks == 0 and r.launches < L
        assert [net.active_count(l) for l in range(L)] == [len(a) for a in ref["active_ids"]]
        cats = net.categories()
        assert np.array_equal(cats, ref["categories"])
        assert same_floats(net.activations(cats), ref["y"])
        dead = np.setdiff1d(np.arange(B), cats)[:64].astype(np.int32)
        assert not net.activations(dead).any()
        # a persistent launch that stops in the middle of the network, continued layer by layer and by another one
        net.run(prune=prune, first_layer=0, n_layers=10, fuse_layers=fuse)
        net.run(prune=prune, first_layer=10, n_layers=4, fuse_layers=1)
        net.run(prune=prune, first_layer=14, n_layers=L - 14, fuse_layers=fuse)
        assert np.array_equal(net.categories(), ref["categories"])
        assert same_floats(net.activations(cats), ref["y"])
        # left to the library (fuse_layers = 0): launches this small stay one per layer
        r = net.run(prune=False, collect_counts=True)
        assert r.persistent_launches == 0 and r.launches == L
        assert [net.active_count(l) for l in range(L)] == [len(a) for a in ref["active_ids"]]
        assert same_floats(net.activations(cats), ref["y"])


@pytest.mark.parametrize("N,L,bias,band_resident", [(1024, 120, -0.3, 1), (1024, 120, -0.3, 0), (4096, 40, -0.35, 1)])
def test_several_layers_per_launch_by_default_at_full_batch(gc, orc, monkeypatch, N, L, bias, band_resident):
    """Batch 60000: left to the library (fuse_layers = 0) the band layers of these widths share launches - resident
    ones up to 1024 neurons (16 rows of a workgroup in LDS through the layers), persistent ones above or when the
    resident form is switched off (one unit queue per XCD, the hand-over between layers inside the XCD's L2).  Every
    activation of every row after the last layer, the per-layer counts and the categories must equal those of one
    launch per layer bit for bit, on live data (rows that survive every layer), pruned and unpruned; an oracle row
    sample pins both."""
    B, S = 60000, 256
    monkeypatch.setenv("SPDNN_BAND_RESIDENT", str(band_resident))
    resident = band_resident and N <= 1024
    print("several layers per launch by default N=%d L=%d resident=%d" % (N, L, resident), flush=True)
    layers = [orc.gen_layer_csr(0, l, N) for l in range(L)]
    ref = orc.infer(orc.gen_features(0, N, 0, S, 0.10, 0.70), layers, bias, prune=False, keep={L - 1})
    rows = np.arange(B, dtype=np.int32)
    with gc.Network(N, B, L, bias=bias) as net:
        net.synth_layers(0)
        net.inspect()
        net.synth_features(0, B, 0.10, 0.70)

        def state():
            acts = np.concatenate([net.activations(rows[i:i + 8192]) for i in range(0, B, 8192)])
            return acts, [net.active_count(l) for l in range(L)], net.categories()

        r1 = net.run(prune=False, collect_counts=True, fuse_layers=1)
        want = state()
        assert r1.persistent_launches == 0 and len(want[2]) > 1000
        assert same_floats(want[0][:S], ref["kept"][L - 1][1])
        for attempt in range(3):
            r = net.run(prune=False, collect_counts=True)
            assert (r.resident_launches if resident else r.persistent_launches) >= 1 and r.persistent_fallbacks == 0 and r.launches < L
            assert (r.persistent_launches if resident else r.resident_launches) == 0
            got = state()
            assert np.array_equal(got[0], want[0]) and got[1] == want[1] and np.array_equal(got[2], want[2]), attempt
        r = net.run(prune=True, collect_counts=True)
        got = state()
        assert np.array_equal(got[0], want[0]) and got[1] == want[1] and np.array_equal(got[2], want[2])


@pytest.mark.parametrize("mode", ["one-queue", "xcd-queues"])
@pytest.mark.parametrize("prune", [True, False])
def test_persistent_launch_that_gives_up(gc, orc, prune, mode, monkeypatch):
    """A unit of a persistent launch waits for its row block for a bounded time only.  With the limit at zero the
    launch gives up at the first look that finds a row block not ready: every workgroup leaves, the host reads how
    far each row block got and finishes the layers with per-layer launches.  Results must not change."""
    for k, v in PERSIST_MODES[mode].items():
        monkeypatch.setenv(k, v)
    monkeypatch.setenv("SPDNN_BAND_RESIDENT", "0")
    N, L, B = 1024, 20, 2600
    print("persistent launch gives up prune=%s %s" % (prune, mode), flush=True)
    layers = [orc.gen_layer_csr(6, l, N) for l in range(L)]
    feats = orc.gen_features(6, N, 0, B, 0.10, 0.55)
    ref = orc.infer(feats, layers, -0.3, prune=True)
    with gc.Network(N, B, L) as net:
        net.synth_layers(6)
        net.inspect()
        net.set_features_dense(feats)
        gave_up = 0
        for attempt in range(3):
            r = net.run(prune=prune, collect_counts=True, fuse_layers=8, persist_wait_us=-1)
            gave_up += r.persistent_fallbacks
            assert r.layers_run == L
            assert [net.active_count(l) for l in range(L)] == [len(a) for a in ref["active_ids"]]
            cats = net.categories()
            assert np.array_equal(cats, ref["categories"])
            assert same_floats(net.activations(cats), ref["y"])
        assert gave_up >= 1
        # and the next run, with the default limit, is persistent again
        r = net.run(prune=prune, collect_counts=True, fuse_layers=8)
        assert r.persistent_launches >= 2 and r.persistent_fallbacks == 0
        assert np.array_equal(net.categories(), ref["categories"])
        assert same_floats(net.activations(cats), ref["y"])


@pytest.mark.parametrize("N,B,kind", [(256, 300, "radix"), (1024, 2100, "radix"), (1024, 700, "hub"), (4096, 1300, "radix")])
def test_resident_launches(gc, orc, N, B, kind):
    """RadiX-Net-like layers of one exact weight, up to 4096 neurons wide, run as resident launches: a workgroup keeps
    16 or 4 rows (by the width) in LDS through all layers of the launch.  Per-layer counts, categories and activations against
    the oracle, pruned and unpruned, whole and cut into calls, and the state after every layer; `hub` layers have
    groups of fewer than 32 inputs."""
    print("resident launches N=%d B=%d %s" % (N, B, kind), flush=True)
    rng = np.random.default_rng(N + B)
    nst = int(np.log2(N)) - 4
    if kind == "hub":
        base = [hub_block_csr(rng, N) for _ in range(3)]
    else:
        base = [radix_like_csr(rng, N, 16 << k) for k in range(nst)]
    L = 2 * len(base) + 1
    layers = [base[l % len(base)] for l in range(L)]
    dens = np.where(rng.random(B) < 0.3, 0.7, 0.08).astype(np.float32)
    feats = (rng.random((B, N), dtype=np.float32) < dens[:, None]).astype(np.float32)
    bias = -0.3 if N <= 1024 else -0.35 if N <= 4096 else -0.4
    ref = orc.infer(feats, layers, bias, prune=True, keep=set(range(L)))
    want_counts = [len(a) for a in ref["active_ids"]]
    assert 0 < want_counts[-1] < B
    with gc.Network(N, B, L, bias=bias) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        net.set_features_dense(feats)
        cats = ref["categories"]
        for prune in (True, False):
            for fuse in (0, 5, 1):
                r = net.run(prune=prune, collect_counts=True, fuse_layers=fuse)
                assert r.layers_run == L
                assert r.persistent_launches == 0 and (r.resident_launches == 0) == (fuse == 1) or (fuse == 0 and prune)
                if fuse == 5:
                    assert r.resident_launches == L // 5 + (1 if L % 5 >= 2 else 0) and r.launches == (L + 4) // 5
                assert [net.active_count(l) for l in range(L)] == want_counts
                assert np.array_equal(net.categories(), cats)
                assert same_floats(net.activations(cats), ref["y"])
                dead = np.setdiff1d(np.arange(B), cats)[:64].astype(np.int32)
                assert not net.activations(dead).any()
        for l in range(1, L, 2):    # the state after layer l, from a resident launch that ends there
            net.run(prune=True, first_layer=0, n_layers=l + 1, fuse_layers=L)
            gid, y = ref["kept"][l]
            assert np.array_equal(net.categories(), ref["active_ids"][l])
            assert same_floats(net.activations(gid), y)
        # cut into calls: resident, layer by layer, resident again (odd and even layer counts)
        net.run(prune=True, first_layer=0, n_layers=3, fuse_layers=3)
        net.run(prune=True, first_layer=3, n_layers=1, fuse_layers=1)
        r = net.run(prune=False, first_layer=4, n_layers=L - 4, collect_counts=True, fuse_layers=L)
        assert r.resident_launches == 1
        assert [net.active_count(l) for l in range(4, L)] == want_counts[4:]
        assert np.array_equal(net.categories(), cats)
        assert same_floats(net.activations(cats), ref["y"])


@pytest.mark.parametrize("N,B,values", [(512, 900, "general"), (1024, 1500, "general"), (1024, 700, "pow2"), (2048, 600, "general"),
                                        (4096, 400, "general")])
def test_resident_launches_of_unstructured_layers(gc, orc, N, B, values):
    """Layers without structure (TILED class) up to 4096 neurons wide run as resident launches too: the 16, 8 or 4 rows of
    a workgroup stay in LDS through the layers, every thread computing whole outputs from its entry list.  Per-layer
    counts, categories and activations against the oracle, pruned and unpruned, whole and cut into calls, and the
    state after every layer."""
    print("resident launches, unstructured layers N=%d B=%d %s" % (N, B, values), flush=True)
    rng = np.random.default_rng(N + B)
    L = 7
    base = [random_csr(rng, N, rng.integers(0, 25, size=N), values) for _ in range(3)]
    layers = [base[l % 3] for l in range(L)]
    dens = np.where(rng.random(B) < 0.3, 0.9, 0.05).astype(np.float32)
    feats = ((rng.random((B, N), dtype=np.float32) < dens[:, None]) * rng.uniform(0.5, 2.0, size=(B, N))).astype(np.float32)
    bias = -0.05
    ref = orc.infer(feats, [sort_rows(c) for c in layers], bias, prune=True, keep=set(range(L)))
    want_counts = [len(a) for a in ref["active_ids"]]
    with gc.Network(N, B, L, bias=bias) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert all(net.layer_plan(l).kernel == gc.KERNEL_TILED for l in range(L))
        net.set_features_dense(feats)
        cats = ref["categories"]
        for prune in (True, False):
            for fuse in (0, 3, 1):
                r = net.run(prune=prune, collect_counts=True, fuse_layers=fuse)
                assert r.layers_run == L and r.persistent_launches == 0
                if fuse == 1:
                    assert r.resident_launches == 0
                elif fuse == 3 or (N <= 1024 and not prune):   # (left to the library, 8- and 4-row workgroups want 8 layers and more)
                    assert r.resident_launches >= 1
                assert [net.active_count(l) for l in range(L)] == want_counts
                assert np.array_equal(net.categories(), cats)
                assert same_floats(net.activations(cats), ref["y"])
        for l in range(L):    # the state after layer l, from a resident launch that ends there
            net.run(prune=True, first_layer=0, n_layers=l + 1, fuse_layers=L)
            gid, y = ref["kept"][l]
            assert np.array_equal(net.categories(), ref["active_ids"][l])
            assert same_floats(net.activations(gid), y)
        net.run(prune=True, first_layer=0, n_layers=3, fuse_layers=3)
        r = net.run(prune=False, first_layer=3, n_layers=L - 3, collect_counts=True, fuse_layers=L)
        assert r.resident_launches == 1
        assert [net.active_count(l) for l in range(3, L)] == want_counts[3:]
        assert np.array_equal(net.categories(), cats)
        assert same_floats(net.activations(cats), ref["y"])


@pytest.mark.parametrize("N,B,K,values,rl", [(1024, 1500, 32, "uniform", 4), (1024, 700, 32, "general", 2), (512, 900, 16, "pow2", 4),
                                             (256, 300, 8, "general", 1), (768, 520, 32, "uniform", 4), (1024, 400, 12, "pow2", 4)])
def test_resident_launches_of_band_layers(gc, orc, monkeypatch, N, B, K, values, rl):
    """BAND layers up to 1024 neurons wide run as resident launches in their QUAD form: 16 rows of a workgroup stay in
    LDS through the layers, a thread computes four neighbouring outputs of the band for four rows from one merged
    step list.  Per-layer counts, categories and activations against the oracle, pruned and unpruned, whole and cut
    into calls, the state after every layer, and the same run with one launch per layer."""
    print("resident launches, band layers N=%d B=%d K=%d %s rl=%d" % (N, B, K, values, rl), flush=True)
    monkeypatch.setenv("SPDNN_ROWS_PER_LANE", str(rl))
    rng = np.random.default_rng(N + B + K)
    L = 9
    layers = []
    for l in range(L):
        rp, c, v = orc.gen_layer_csr(11, l, N, K)
        if values == "pow2":
            v = np.ldexp(1.0, rng.integers(-5, -2, size=len(v)) + (2 if K <= 16 else 0)).astype(np.float32)
        elif values == "general":
            v = (rng.uniform(-0.05, 0.2, size=len(v)) * (32.0 / K)).astype(np.float32)
        else:
            v = np.full(len(v), 2.0 / K, dtype=np.float32)
        layers.append((rp, c, v))
    dens = np.where(rng.random(B) < 0.4, 0.8, 0.05).astype(np.float32)
    feats = ((rng.random((B, N), dtype=np.float32) < dens[:, None]) * rng.uniform(0.5, 2.0, size=(B, N))).astype(np.float32)
    bias = -0.3
    ref = orc.infer(feats, layers, bias, prune=True, keep=set(range(L)))
    want_counts = [len(a) for a in ref["active_ids"]]
    assert 0 < want_counts[-1] < B, want_counts
    with gc.Network(N, B, L, bias=bias) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert all(net.layer_plan(l).kernel == gc.KERNEL_BAND for l in range(L))
        net.set_features_dense(feats)
        cats = ref["categories"]
        for prune in (True, False):
            for fuse in (0, 4, 1):
                r = net.run(prune=prune, collect_counts=True, fuse_layers=fuse)
                assert r.layers_run == L
                if fuse == 1:
                    assert r.resident_launches == 0
                elif fuse == 4 or not prune:
                    assert r.resident_launches >= 1 and r.persistent_launches == 0
                assert [net.active_count(l) for l in range(L)] == want_counts
                assert np.array_equal(net.categories(), cats)
                assert same_floats(net.activations(cats), ref["y"])
        for l in range(L):    # the state after layer l, from a resident launch that ends there
            net.run(prune=True, first_layer=0, n_layers=l + 1, fuse_layers=L)
            gid, y = ref["kept"][l]
            assert np.array_equal(net.categories(), ref["active_ids"][l])
            assert same_floats(net.activations(gid), y)
        net.run(prune=True, first_layer=0, n_layers=3, fuse_layers=3)
        r = net.run(prune=False, first_layer=3, n_layers=L - 3, collect_counts=True, fuse_layers=L)
        assert r.resident_launches == 1
        assert [net.active_count(l) for l in range(3, L)] == want_counts[3:]
        assert np.array_equal(net.categories(), cats)
        assert same_floats(net.activations(cats), ref["y"])


def test_resident_launches_full_batch(gc, orc):
    """Batch 60000 of RadiX-Net-like layers, N=1024: every activation of every row, the per-layer counts and the
    categories of the default run (resident launches) equal those of one launch per layer bit for bit, on live
    data, pruned and unpruned; an oracle row sample pins both."""
    N, L, B, S, bias = 1024, 30, 60000, 256, -0.3
    print("resident launches, full batch", flush=True)
    rng = np.random.default_rng(5)
    base = [radix_like_csr(rng, N, 16 << k) for k in range(6)]
    layers = [base[l % 6] for l in range(L)]
    dens = np.where(rng.random(B) < 0.3, 0.7, 0.08).astype(np.float32)
    feats = (rng.random((B, N), dtype=np.float32) < dens[:, None]).astype(np.float32)
    ref = orc.infer(feats[:S], layers, bias, prune=False, keep={L - 1})
    rows = np.arange(B, dtype=np.int32)
    with gc.Network(N, B, L, bias=bias) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        net.set_features_dense(feats)

        def state():
            acts = np.concatenate([net.activations(rows[i:i + 8192]) for i in range(0, B, 8192)])
            return acts, [net.active_count(l) for l in range(L)], net.categories()

        r1 = net.run(prune=False, collect_counts=True, fuse_layers=1)
        want = state()
        assert r1.resident_launches == 0 and len(want[2]) > 1000
        assert same_floats(want[0][:S], ref["kept"][L - 1][1])
        for prune in (False, True):
            r = net.run(prune=prune, collect_counts=True)
            assert r.resident_launches >= 1
            got = state()
            assert np.array_equal(got[0], want[0]) and got[1] == want[1] and np.array_equal(got[2], want[2]), prune


@pytest.mark.parametrize("rl", [1, 2])
def test_persistent_launches_on_buffers_that_stay_in_l1(gc, orc, rl, monkeypatch):
    """Narrow layers in small row blocks: the buffers of a persistent launch stay in the CUs' L1 from layer to layer, so a
    unit that does not really invalidate its L1 reads what the buffer held two layers earlier (found by a random case:
    the workgroup-scope invalidate is no invalidate outside threadgroup-split mode).  Three and four layers per launch,
    one unit queue per XCD, pruned: counts, categories and activations against the oracle, several networks, each run
    three times."""
    monkeypatch.setenv("SPDNN_ROWS_PER_LANE", str(rl))
    monkeypatch.setenv("SPDNN_PERSIST_XCD", "1")
    monkeypatch.setenv("SPDNN_BAND_RESIDENT", "0")
    N, B = 256, 1500
    for seed in range(8):
        rng = np.random.default_rng(9100 + seed)
        L = 3 + seed % 2
        layers = []
        for l in range(L):
            rp, c, v = orc.gen_layer_csr(int(rng.integers(0, 1000)), l, N, 4)
            layers.append((rp, c, rng.uniform(-0.1, 0.2, size=len(v)).astype(np.float32)))
        feats = (rng.uniform(0, 3, size=(B, N)) * (rng.random((B, N)) < 0.8)).astype(np.float32)
        ref = orc.infer(feats, layers, -0.05, prune=True)
        want_counts = [len(a) for a in ref["active_ids"]]
        with gc.Network(N, B, L, bias=-0.05) as net:
            for l, csr in enumerate(layers):
                net.set_layer_csr(l, *csr)
            net.inspect()
            net.set_features_dense(feats)
            for rep in range(3):
                r = net.run(prune=True, collect_counts=True, fuse_layers=L)
                assert r.persistent_launches == 1 and r.persistent_fallbacks == 0
                assert [net.active_count(l) for l in range(L)] == want_counts, (seed, rep)
                assert np.array_equal(net.categories(), ref["categories"]), (seed, rep)
                assert same_floats(net.activations(ref["categories"]), ref["y"]), (seed, rep)


@pytest.mark.parametrize("mode", ["one-queue", "xcd-queues-light"])
@pytest.mark.parametrize("N,B,values", [(1024, 2100, "uniform"), (1024, 900, "general"), (4096, 1300, "uniform")])
def test_persistent_launches_block_kernel(gc, orc, N, B, values, mode, monkeypatch):
    """RadiX-Net-like layers on the BLOCK kernel (narrow layers, and the BLOCK form of run chains on small batches),
    several layers per launch: bit-equal to the oracle, pruned and unpruned, and to one launch per layer."""
    for k, v in PERSIST_MODES[mode].items():
        monkeypatch.setenv(k, v)
    monkeypatch.setenv("SPDNN_RESIDENT", "0")    # (layers of one exact weight would otherwise run as resident launches)
    print("persistent BLOCK launches N=%d B=%d %s %s" % (N, B, values, mode), flush=True)
    rng = np.random.default_rng(N + B)
    nst = int(np.log2(N)) - 4
    base = [radix_like_csr(rng, N, 16 << k, values) for k in range(nst)]
    L = 2 * nst + 1
    layers = [base[l % nst] for l in range(L)]
    dens = np.where(rng.random(B) < 0.3, 0.7, 0.08).astype(np.float32)
    feats = (rng.random((B, N), dtype=np.float32) < dens[:, None]).astype(np.float32)
    bias = -0.3 if N == 1024 else -0.35
    ref = orc.infer(feats, layers, bias, prune=True)
    with gc.Network(N, B, L, bias=bias) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        net.set_features_dense(feats)
        for prune in (True, False):
            r = net.run(prune=prune, collect_counts=True, fuse_layers=6)
            assert r.persistent_launches >= 1 and r.persistent_fallbacks == 0
            assert [net.active_count(l) for l in range(L)] == [len(a) for a in ref["active_ids"]]
            cats = net.categories()
            assert np.array_equal(cats, ref["categories"])
            assert same_floats(net.activations(cats), ref["y"])
        r = net.run(prune=True, collect_counts=True, fuse_layers=6, persist_wait_us=-1)
        assert np.array_equal(net.categories(), ref["categories"])
        assert same_floats(net.activations(cats), ref["y"])


@pytest.mark.parametrize("values", ["uniform", "pow2", "general"])
@pytest.mark.parametrize("N,B", [(1024, 1500), (4096, 700)])
def test_fused_pairs_in_lds(gc, orc, monkeypatch, N, B, values):
    """Layers that are bands over one common neuron order run two per launch, the activations between
    them kept in LDS (the reference's fused kernel, src/microbenchmark/fuse.cu:16-110): counts of every
    layer - the one inside a pair included -, categories and activations must be the oracle's, with
    and without pruning, and the same as with every layer in its own launch."""
    monkeypatch.setenv("SPDNN_BAND_RESIDENT", "0")   # (bands up to 1024 neurons would share resident launches: the pairs are for wider ones)
    print("fused pairs N=%d B=%d %s" % (N, B, values), flush=True)
    rng = np.random.default_rng(N + B)
    L = 7
    perm = rng.permutation(N)
    layers = [common_band_csr(rng, N, perm, values) for _ in range(L)]
    feats = orc.gen_features(8, N, 0, B, 0.10, 0.60)
    ref = orc.infer(feats, layers, -0.3, prune=True, keep=set(range(L)))
    want_counts = [len(a) for a in ref["active_ids"]]
    assert want_counts[-1] > 0 and want_counts[-1] < B
    with gc.Network(N, B, L, bias=-0.3) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert [net.layer_plan(l).fuse_next for l in range(L)] == [1] * (L - 1) + [0]
        net.set_features_dense(feats)
        cats = ref["categories"]
        for prune in (True, False):
            for fuse in (2, 0):
                r = net.run(prune=prune, collect_counts=True, fuse_layers=fuse)
                assert r.layers_run == L
                assert (r.fused_pairs, r.launches) == ((3, 4) if fuse == 2 else (0, L))
                assert [net.active_count(l) for l in range(L)] == want_counts
                assert np.array_equal(net.categories(), cats)
                assert same_floats(net.activations(cats), ref["y"])
                dead = np.setdiff1d(np.arange(B), cats)[:64].astype(np.int32)
                assert not net.activations(dead).any()
        # stops and continuations that cut pairs differently: (0,1) 2 | (3,4) (5,6) and (0,1) (2,3) | 4 (5,6)
        for cut in (3, 4, 1):
            net.run(prune=True, first_layer=0, n_layers=cut, fuse_layers=2)
            gid, y = ref["kept"][cut - 1]
            assert np.array_equal(net.categories(), ref["active_ids"][cut - 1])
            assert same_floats(net.activations(gid), y)
            r = net.run(prune=False, first_layer=cut, n_layers=L - cut, collect_counts=True, fuse_layers=2)
            assert r.fused_pairs == (L - cut) // 2
            assert [net.active_count(l) for l in range(cut, L)] == want_counts[cut:]
            assert np.array_equal(net.categories(), cats)
            assert same_floats(net.activations(cats), ref["y"])


def test_fused_pairs_radix_common(gc, orc, monkeypatch):
    """RadiX-Net layers behind one hidden neuron numbering (strides 16, 32, 64, ...): the layers of stride
    16 and 32 take the network's common order and neighbours among them run as one launch with the
    activations in LDS.  Counts of every layer, categories and activations against the oracle, pruned
    and not, fused and one launch per layer; then the full batch: an oracle row sample, and the whole
    batch against the run with one launch per layer."""
    N, B = 4096, 700
    print("fused pairs, radix layers of one numbering N=%d B=%d" % (N, B), flush=True)
    rng = np.random.default_rng(N + B)
    perm = rng.permutation(N)
    strides = [16, 32, 64, 16, 32, 32, 16, 128]
    L = len(strides)
    layers = [radix_like_csr(rng, N, s, perm=perm) for s in strides]
    feats = orc.gen_features(8, N, 0, B, 0.10, 0.60)
    ref = orc.infer(feats, layers, -0.4, prune=True, keep=set(range(L)))
    want_counts = [len(a) for a in ref["active_ids"]]
    assert 0 < want_counts[-1] < B
    monkeypatch.setenv("SPDNN_BLOCK_FORM_MAX_ELEMS", "0")   # a batch this small would run the layers' BLOCK form
    monkeypatch.setenv("SPDNN_RESIDENT", "0")   # and layers this narrow as resident launches (the pairs are for wider ones)
    with gc.Network(N, B, L, bias=-0.4) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert [net.layer_plan(l).common_order for l in range(L)] == [1, 2, 0, 1, 2, 2, 1, 0]
        assert [net.layer_plan(l).fuse_next for l in range(L)] == [1, 0, 0, 1, 1, 1, 0, 0]
        net.set_features_dense(feats)
        cats = ref["categories"]
        for prune in (True, False):
            for fuse in (2, 1):
                r = net.run(prune=prune, collect_counts=True, fuse_layers=fuse)
                assert r.layers_run == L
                assert (r.fused_pairs, r.launches) == ((3, 5) if fuse == 2 else (0, L))
                assert [net.active_count(l) for l in range(L)] == want_counts
                assert np.array_equal(net.categories(), cats)
                assert same_floats(net.activations(cats), ref["y"])
        for l in range(L):    # every layer's survivors and their activations, the layer inside a pair included
            net.run(prune=True, first_layer=0, n_layers=l + 1, fuse_layers=2)
            gid, y = ref["kept"][l]
            assert np.array_equal(net.categories(), ref["active_ids"][l])
            assert same_floats(net.activations(gid), y)
    monkeypatch.delenv("SPDNN_BLOCK_FORM_MAX_ELEMS")
    B, S = 60000, 768
    print("fused pairs, radix layers of one numbering N=%d B=%d" % (N, B), flush=True)
    ref = orc.infer(orc.gen_features(9, N, 0, S, 0.10, 0.60), layers, -0.4, prune=True)
    with gc.Network(N, B, L, bias=-0.4) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        net.synth_features(9, B, 0.10, 0.60)
        r = net.run(prune=False, collect_counts=True)     # left to the library, launches of this size run the pairs fused
        assert r.fused_pairs == 3 and r.launches == 5
        counts = [net.active_count(l) for l in range(L)]
        cats = net.categories()
        assert np.array_equal(cats[cats < S], ref["categories"])
        assert same_floats(net.activations(ref["categories"]), ref["y"])
        probe = cats[:: max(1, len(cats) // 512)].astype(np.int32)
        y_fused = net.activations(probe)
        net.synth_features(9, B, 0.10, 0.60)
        r = net.run(prune=False, collect_counts=True, fuse_layers=1)
        assert r.fused_pairs == 0
        assert [net.active_count(l) for l in range(L)] == counts
        assert np.array_equal(net.categories(), cats)
        assert same_floats(net.activations(probe), y_fused)


def test_fused_pairs_full_batch(gc, orc):
    """The fused pair on a batch of 60000 (235 row blocks, several segments per row block, streaming
    loads and stores): an oracle row sample through 6 layers, and the whole batch against the run
    with one launch per layer."""
    N, B, L, S = 4096, 60000, 6, 768
    print("fused pairs, full batch", flush=True)
    rng = np.random.default_rng(77)
    perm = rng.permutation(N)
    layers = [common_band_csr(rng, N, perm, "uniform") for _ in range(L)]
    ref = orc.infer(orc.gen_features(9, N, 0, S, 0.10, 0.60), layers, -0.35, prune=True)
    with gc.Network(N, B, L, bias=-0.35) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        net.synth_features(9, B, 0.10, 0.60)
        r = net.run(prune=True, collect_counts=True, fuse_layers=2)
        assert r.fused_pairs == 3 and r.launches == 3
        counts = [net.active_count(l) for l in range(L)]
        cats = net.categories()
        assert np.array_equal(cats[cats < S], ref["categories"])
        assert same_floats(net.activations(ref["categories"]), ref["y"])
        probe = cats[:: max(1, len(cats) // 512)].astype(np.int32)
        y_fused = net.activations(probe)
        net.run(prune=False, collect_counts=True, fuse_layers=1)
        assert [net.active_count(l) for l in range(L)] == counts
        assert np.array_equal(net.categories(), cats)
        assert same_floats(net.activations(probe), y_fused)
        # left to the library (fuse_layers = 0) a launch of this size runs the pairs fused; a pruned run only while
        # enough rows are left (here: after the first compaction it goes on with one launch per layer)
        net.synth_features(9, B, 0.10, 0.60)
        r = net.run(prune=False, collect_counts=True)
        assert (r.fused_pairs, r.launches) == (3, 3)
        assert [net.active_count(l) for l in range(L)] == counts
        assert same_floats(net.activations(probe), y_fused)
        net.synth_features(9, B, 0.10, 0.60)
        r = net.run(prune=True, collect_counts=True)
        assert 1 <= r.fused_pairs <= 3 and r.launches == L - r.fused_pairs
        assert [net.active_count(l) for l in range(L)] == counts
        assert np.array_equal(net.categories(), cats)
        assert same_floats(net.activations(probe), y_fused)
    with gc.Network(N, 512, L, bias=-0.35) as net:      # 2^21 elements: two launches are faster, and are what runs
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        net.synth_features(9, 512, 0.10, 0.60)
        r = net.run(prune=False, collect_counts=True)
        assert (r.fused_pairs, r.launches) == (0, L)
        assert [net.active_count(l) for l in range(L)] == [len(a) for a in orc.infer(orc.gen_features(9, N, 0, 512, 0.10, 0.60), layers, -0.35, prune=False)["active_ids"]]


def test_fused_pairs_several_segments_per_row_block(gc, orc, monkeypatch):
    """A pruned run in which a row block's band is cut into segments that run one after the other (more
    workgroups than the chip holds): a workgroup that starts late finds rows already stamped by the
    segments that have finished, and must still see them as alive."""
    monkeypatch.setenv("SPDNN_PAIR_SEGLEN", "512")
    N, B, L, S = 4096, 60000, 7, 512
    print("fused pairs, segments in several rounds", flush=True)
    rng = np.random.default_rng(78)
    perm = rng.permutation(N)
    # weights of both signs with gain above 1 and dense rows: every row stays alive for good (so that no row of
    # a row block dies in a pair), at values below the clamp that differ from layer to layer
    layers = []
    for _ in range(L):
        rp, c, v = common_band_csr(rng, N, perm, "general")
        layers.append((rp, c, rng.uniform(-0.3, 0.4, size=len(v)).astype(np.float32)))
    ref = orc.infer(orc.gen_features(10, N, 0, S, 0.30, 0.90), layers, -0.35, prune=True)
    assert len(ref["categories"]) == S and float(np.median(ref["y"])) < 16.0
    with gc.Network(N, B, L, bias=-0.35) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        net.synth_features(10, B, 0.30, 0.90)
        net.run(prune=False, collect_counts=True, fuse_layers=1)
        counts = [net.active_count(l) for l in range(L)]
        cats = net.categories()
        assert np.array_equal(cats[cats < S], ref["categories"])
        # layer 0 alone, then the pairs (1,2), (3,4), ...: every pair runs behind a stamped layer
        net.run(prune=True, first_layer=0, n_layers=1)
        r = net.run(prune=True, first_layer=1, n_layers=L - 1, collect_counts=True, fuse_layers=2)
        assert r.fused_pairs == (L - 1) // 2
        assert [net.active_count(l) for l in range(1, L)] == counts[1:]
        assert np.array_equal(net.categories(), cats)
        assert same_floats(net.activations(ref["categories"]), ref["y"])


@pytest.mark.parametrize("kind", ["band", "radix", "radix-blocks", "hub", "irregular", "irregular-gather"])
def test_pruned_run_with_rows_that_never_die(gc, orc, kind, monkeypatch):
    """Full batch, pruning on, and every row alive for good at values below the clamp that differ from layer
    to layer: a workgroup that wrongly takes its rows for dead (rows that the workgroups before it have
    already stamped) leaves another layer's values behind, which this data shows."""
    from helpers import hub_block_csr, radix_like_csr
    N, B, L, S = 4096, 60000, 6, 256
    print("rows that never die:", kind, flush=True)
    if kind == "radix-blocks":
        monkeypatch.setenv("SPDNN_RUN_CHAINS_MIN_N", "0")
    rng = np.random.default_rng(5)

    def layer(l):
        if kind == "band":
            rp, c, v = orc.gen_layer_csr(3, l, N)
        elif kind.startswith("radix"):
            rp, c, v = radix_like_csr(rng, N, (16, 256, 2048)[l % 3], "general")
        elif kind == "hub":
            rp, c, v = hub_block_csr(rng, N, "general")
        else:
            rp, c, v = sort_rows(random_csr(rng, N, 32, "general"))   # (the oracle adds in the order given)
        return rp, c, rng.uniform(-0.3, 0.4, size=len(v)).astype(np.float32)

    layers = [layer(l) for l in range(L)]
    ref = orc.infer(orc.gen_features(10, N, 0, S, 0.30, 0.90), layers, -0.35, prune=True, keep={2})
    assert len(ref["active_ids"][-2]) == S and 1.0 < float(np.median(ref["y"])) < 16.0
    want = {"band": gc.KERNEL_BAND, "radix": gc.KERNEL_BAND, "radix-blocks": gc.KERNEL_BLOCK, "hub": gc.KERNEL_BLOCK,
            "irregular": gc.KERNEL_TILED, "irregular-gather": gc.KERNEL_GATHER}[kind]
    force = gc.KERNEL_GATHER if kind == "irregular-gather" else gc.KERNEL_AUTO
    with gc.Network(N, B, L, bias=-0.35, force_kernel=force) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert all(net.layer_plan(l).kernel == want for l in range(L))
        net.synth_features(10, B, 0.30, 0.90)
        # three layers, then the rest in a second call: both begin behind stamped rows after the first layer
        net.run(prune=True, first_layer=0, n_layers=3, collect_counts=True)
        ids, y = ref["kept"][2]
        assert np.array_equal(net.categories()[: len(ids)], ids)
        assert same_floats(net.activations(ids), y)
        net.run(prune=True, first_layer=3, n_layers=L - 3, collect_counts=True)
        cats = net.categories()
        assert np.array_equal(cats[cats < S], ref["categories"])
        assert same_floats(net.activations(ref["categories"]), ref["y"])
        pruned = [net.active_count(l) for l in range(L)]
        net.synth_features(10, B, 0.30, 0.90)
        net.run(prune=False, collect_counts=True)
        assert [net.active_count(l) for l in range(L)] == pruned
        assert np.array_equal(net.categories(), cats)


def test_persistent_launches_when_everything_dies(gc, orc, monkeypatch):
    """Literal inputs: all rows die within a few layers; the units of dead row blocks are skipped."""
    monkeypatch.setenv("SPDNN_BAND_RESIDENT", "0")
    N, L, B = 1024, 40, 2000
    print("persistent launches, all rows die", flush=True)
    layers = [orc.gen_layer_csr(0, l, N) for l in range(12)]
    ref = orc.infer(orc.gen_features(0, N, 0, B), layers, -0.3, prune=True)
    want = [len(a) for a in ref["active_ids"]] + [0] * (L - 12)
    with gc.Network(N, B, L) as net:
        net.synth_layers(0)
        net.inspect()
        net.synth_features(0, B)
        for prune in (True, False):
            r = net.run(prune=prune, collect_counts=True, fuse_layers=8)
            assert [net.active_count(l) for l in range(L)] == want
            assert r.active_rows == 0 and len(net.categories()) == 0
            assert not net.activations(np.arange(50, dtype=np.int32)).any()


@pytest.mark.parametrize("chains", [True, False])
@pytest.mark.parametrize("values", ["uniform", "pow2", "general"])
def test_block_kernel_radix_like_layers(gc, orc, values, chains, monkeypatch):
    """RadiX-Net-like layers (16 outputs sharing two 16-wide input runs, hidden behind random
    relabellings) are walked as chains by the band kernel; groups without a chain go to the BLOCK
    kernel; mixed with a circulant band layer and an irregular layer."""
    from helpers import hub_block_csr, radix_like_csr
    N, B = 1024, 300
    print("block kernel values=%s chains=%s" % (values, chains), flush=True)
    if chains:   # by default widths below 4096 stay on the BLOCK kernel, and small batches take the BLOCK form
        monkeypatch.setenv("SPDNN_RUN_CHAINS_MIN_N", "256")
        monkeypatch.setenv("SPDNN_BLOCK_FORM_MAX_ELEMS", "0")
    rk, rh = (gc.KERNEL_BAND, 32) if chains else (gc.KERNEL_BLOCK, -1)
    rng = np.random.default_rng(17)
    layers = [radix_like_csr(rng, N, 16 << l, values) for l in range(4)]
    layers.append(orc.gen_layer_csr(3, 0, N))                                  # BAND
    layers.append(radix_like_csr(rng, N, 256, values, run=8))                   # groups of 8, 16 inputs
    layers.append(sort_rows(random_csr(rng, N, rng.integers(1, 20, size=N), "pow2")))   # GATHER
    layers.append(hub_block_csr(rng, N, values))                               # 32 inputs, no chain
    layers.append(radix_like_csr(rng, N, 512, values))                          # cycles of two groups
    L = len(layers)
    feats = (rng.uniform(0, 3, size=(B, N)) * (rng.random((B, N)) < 0.4)).astype(np.float32)
    with gc.Network(N, B, L, bias=-0.2) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        kinds = [net.layer_plan(l).kernel for l in range(L)]
        assert kinds == [rk] * 4 + [gc.KERNEL_BAND, gc.KERNEL_BLOCK, gc.KERNEL_TILED, gc.KERNEL_BLOCK, rk]
        assert [net.layer_plan(l).band_halo for l in range(L)] == [rh] * 4 + [31, -1, -1, -1, rh]
        net.set_features_dense(feats)
        _layer_by_layer(gc, orc, net, layers, feats, prune=True)
        ref = orc.infer(feats, layers, -0.2, prune=True)
        for prune in (True, False):
            net.run(prune=prune, collect_counts=True)
            assert [net.active_count(l) for l in range(L)] == [len(a) for a in ref["active_ids"]]
            assert np.array_equal(net.categories(), ref["categories"])


@pytest.mark.parametrize("form", ["band", "block"])
@pytest.mark.parametrize("N,strides", [(4096, (16, 256, 2048)), (65536, (16, 1024, 32768))])
def test_radix_like_layers_at_challenge_widths(gc, orc, N, strides, form, monkeypatch):
    """RadiX-Net-like layers (two 16-wide input runs per group of 16 outputs, first, middle and last
    stride of the width, behind random relabellings) at N=4096 and at the headline width: planned
    as run chains for the band kernel under the default settings, and run in both of their forms -
    the band walk (what large batches get) and the BLOCK form (what small batches get)."""
    from helpers import radix_like_csr
    B = 300
    monkeypatch.setenv("SPDNN_BLOCK_FORM_MAX_ELEMS", "0" if form == "band" else str(1 << 40))
    print("radix-like N=%d strides %s form %s" % (N, strides, form), flush=True)
    rng = np.random.default_rng(N)
    layers = [radix_like_csr(rng, N, st, "uniform") for st in strides]
    L = len(layers)
    feats = (rng.uniform(0, 2, size=(B, N)) * (rng.random((B, N)) < 0.3)).astype(np.float32)
    with gc.Network(N, B, L, bias=-0.3) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        for l in range(L):
            p = net.layer_plan(l)
            assert p.kernel == gc.KERNEL_BAND and p.band_halo == 32 and p.block_form == 1
        net.set_features_dense(feats)
        _layer_by_layer(gc, orc, net, layers, feats, prune=True)


@pytest.mark.parametrize("N,B,L,bias", [(4096, 60000, 6, -0.35), (16384, 60000, 4, -0.4), (65536, 60000, 3, -0.45)])
def test_headline_widths_against_oracle_sample(gc, orc, N, B, L, bias):
    """The wider configurations at full batch, features generated on the device with
    survivor densities; the oracle runs a row sample (rows are independent)."""
    print("wide N=%d B=%d" % (N, B), flush=True)
    S = 384
    layers = [orc.gen_layer_csr(0, l, N) for l in range(L)]
    ref = orc.infer(orc.gen_features(0, N, 0, S, 0.10, 0.60), layers, bias, prune=False, keep=set(range(L)))
    rows = np.arange(S, dtype=np.int32)
    with gc.Network(N, B, L) as net:
        assert net.bias == pytest.approx(bias)
        net.synth_layers(0)
        net.inspect()
        net.synth_features(0, B, 0.10, 0.60)
        for l in range(L):
            net.run(prune=True, first_layer=l, n_layers=1)
            cats = net.categories()
            assert np.array_equal(cats[cats < S], ref["active_ids"][l]), "layer %d" % l
            assert same_floats(net.activations(rows), ref["kept"][l][1]), "layer %d" % l
        full = net.run(prune=False, collect_counts=True)
        paired, candidates, peak = net.feature_placement()
        print("feature buffers paired over two memory regions:", paired, "candidates", candidates, "search peak GiB %.1f" % (peak / 2**30), flush=True)
        assert peak >= 6 * ((B + 255) // 256 * 256 // 2) * N * 4
        assert candidates >= 6      # three buffers of two halves; more candidates = the two-region search ran (N >= 4096 here)
        assert np.array_equal(net.categories()[net.categories() < S], ref["active_ids"][-1])
        assert same_floats(net.activations(rows), ref["kept"][L - 1][1])


@pytest.mark.parametrize("N,L,bias,S", [(4096, 480, -0.35, 512), (16384, 1920, -0.4, 96), (65536, 1920, -0.45, 96)],
                         ids=["cfg2", "cfg3", "cfg4"])
def test_full_depth_cfg2_cfg3_cfg4(gc, orc, N, L, bias, S):
    """N=4096 x 480 layers, N=16384 x 1920 layers and the headline N=65536 x 1920 layers at batch
    60000, every layer, with densities up to 0.7 so that rows survive to the end: pruned run against
    the unpruned run (size-independent, N=4096) and against the oracle on the first S rows through
    all layers (categories inside the sample, and the survivors' activations bit for bit)."""
    B = 60000
    print("full depth N=%d L=%d" % (N, L), flush=True)
    with gc.Network(N, B, L) as net:
        assert net.bias == pytest.approx(bias)
        net.synth_layers(0)
        net.inspect()
        assert all(net.layer_plan(l).kernel == gc.KERNEL_BAND for l in range(0, L, 37))
        net.synth_features(0, B, 0.10, 0.70)
        rp = net.run(prune=True, collect_counts=True)
        counts_p = [net.active_count(l) for l in range(L)]
        cats_p = net.categories()
        sample = cats_p[cats_p < S][:64].astype(np.int32)
        y_p = net.activations(sample)
        if N == 4096:
            net.run(prune=False, collect_counts=True)
            assert counts_p == [net.active_count(l) for l in range(L)]
            assert np.array_equal(cats_p, net.categories())
            assert same_floats(y_p, net.activations(sample))
    print("survivors", counts_p[0], counts_p[-1], "compactions", rp.compactions, flush=True)
    assert counts_p == sorted(counts_p, reverse=True) and 0 < counts_p[-1] < B and rp.compactions >= 1
    assert len(cats_p) == counts_p[-1] and np.array_equal(cats_p, np.sort(cats_p))
    def layer_of(l):
        if l % 240 == 0:
            print("  oracle layer", l, flush=True)    # a long leg (N=65536: about 100 s): keep the log moving
        return orc.gen_layer_csr(0, l, N) if l < L else None

    ref = orc.infer(orc.gen_features(0, N, 0, S, 0.10, 0.70), layer_of, bias, prune=True)
    assert np.array_equal(cats_p[cats_p < S], ref["categories"])
    assert len(sample) > 0 and same_floats(y_p, ref["y"][:len(sample)])


@pytest.mark.parametrize("name,N,L,bias", [("cfg1", 1024, 120, -0.30), ("cfg2", 4096, 480, -0.35),
                                           ("cfg3", 16384, 1920, -0.40), ("cfg4", 65536, 1920, -0.45)])
def test_literal_configs_full_batch(gc, orc, name, N, L, bias):
    """The configurations as written: batch 60000, seed 0, feature density U[0.10, 0.25] per row.
    Every row dies within a few layers, so the final category set is empty and parity is checked
    per layer: for the layers before everything has died, the active ids inside an oracle row
    sample and the sample's activations (bit for bit); afterwards zero rows; and the whole-network
    pruned run must report the same per-layer counts and no categories."""
    B, S, seed = 60000, 2048, 0
    print("literal %s: N=%d L=%d B=%d" % (name, N, L, B), flush=True)
    head = 10                                    # every row is dead long before this layer
    layers = [orc.gen_layer_csr(seed, l, N) for l in range(head)]
    ref = orc.infer(orc.gen_features(seed, N, 0, S, 0.10, 0.25), layers, bias, prune=False, keep=set(range(head)))
    ref_counts = [len(a) for a in ref["active_ids"]]
    assert ref_counts[0] > 0 and ref_counts[-1] == 0, ref_counts
    rows = np.arange(S, dtype=np.int32)
    with gc.Network(N, B, L) as net:
        assert net.bias == pytest.approx(bias)
        net.synth_layers(seed)
        net.inspect()
        net.synth_features(seed, B, 0.10, 0.25)
        step_counts = []
        for l in range(head):
            r = net.run(prune=True, first_layer=l, n_layers=1, collect_counts=True)
            cats = net.categories()
            step_counts.append(len(cats))
            assert r.active_rows == len(cats) and net.active_count(l) == len(cats)
            assert np.array_equal(cats[cats < S], ref["active_ids"][l]), "layer %d" % l
            assert same_floats(net.activations(rows), ref["kept"][l][1]), "layer %d" % l
            if len(cats) == 0:
                break
        assert step_counts[-1] == 0 and step_counts == sorted(step_counts, reverse=True)
        r = net.run(prune=True, collect_counts=True)
        counts = [net.active_count(l) for l in range(L)]
        print("literal %s: active rows per layer %s, layers launched %d" % (name, counts[:len(step_counts)], r.layers_run),
              flush=True)
        assert counts[:len(step_counts)] == step_counts and not any(counts[len(step_counts):])
        assert r.active_rows == 0 and len(net.categories()) == 0 and r.layers_run < L
        assert not net.activations(rows[:64]).any()


def test_unpruned_run_continues_a_pruned_one(gc, orc, monkeypatch):
    """A row block whose rows have all died is skipped by pruned launches and keeps stale values in
    the work buffers.  A run without pruning that continues from there must not bring them back:
    64-row blocks, 65 rows, the last block holds one row that dies at once while the others live."""
    monkeypatch.setenv("SPDNN_ROWS_PER_LANE", "1")
    N, L, B = 256, 8, 65
    rng = np.random.default_rng(4)
    layers = [orc.gen_layer_csr(11, l, N) for l in range(L)]
    feats = (rng.random((B, N)) < 0.6).astype(np.float32) * 2.0
    # the last row is alive after layer 0 and dead after layer 1: layer 1 writes its zeros into one
    # work buffer, the other one keeps the row's nonzero layer-0 output in a block that is skipped from then on
    for _ in range(200):
        cand = (rng.random((1, N)) < 0.2).astype(np.float32)
        probe = orc.infer(cand, layers[:2], -0.3, prune=False)
        if len(probe["active_ids"][0]) == 1 and len(probe["active_ids"][1]) == 0:
            break
    else:
        raise AssertionError("no candidate row dies exactly at layer 1")
    feats[64] = cand[0]
    ref = orc.infer(feats, layers, -0.3, prune=False, keep=set(range(L)))
    assert 64 in ref["active_ids"][0] and 64 not in ref["active_ids"][1] and len(ref["active_ids"][L - 1]) == 64
    rows = np.arange(B, dtype=np.int32)
    for split in (2, 3, 4):
        with gc.Network(N, B, L, bias=-0.3) as net:
            for l, csr in enumerate(layers):
                net.set_layer_csr(l, *csr)
            net.inspect()
            net.set_features_dense(feats)
            r = net.run(prune=True, first_layer=0, n_layers=split, collect_counts=True, compact_threshold=0.01)
            assert r.compactions == 0
            net.run(prune=False, first_layer=split, n_layers=L - split, collect_counts=True)
            assert [net.active_count(l) for l in range(L)] == [len(a) for a in ref["active_ids"]], split
            assert np.array_equal(net.categories(), ref["active_ids"][L - 1]), split
            assert same_floats(net.activations(rows), ref["kept"][L - 1][1]), split


@pytest.mark.parametrize("N,K,B", [(256, 32, 1), (256, 4, 65), (512, 12, 257), (128, 8, 40), (100, 5, 33), (2048, 36, 70)])
def test_small_and_odd_shapes(gc, orc, N, K, B):
    """Smallest band layers, a single row, widths that are not a multiple of 256 and rows longer
    than 32 entries (general kernel)."""
    print("odd shape N=%d K=%d B=%d" % (N, K, B), flush=True)
    L = 3
    layers = [orc.gen_layer_csr(4, l, N, K, 0.0625) for l in range(L)]
    feats = orc.gen_features(4, N, 0, B, 0.2, 0.9)
    with gc.Network(N, B, L, bias=-0.05) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        want = gc.KERNEL_BAND if (N % 256 == 0 and K % 4 == 0 and K <= 32) else gc.KERNEL_TILED
        assert all(net.layer_plan(l).kernel == want for l in range(L))
        net.set_features_dense(feats)
        _layer_by_layer(gc, orc, net, layers, feats, prune=True)
        ref = orc.infer(feats, layers, -0.05, prune=True)
        net.run(prune=True)
        assert np.array_equal(net.categories(), ref["categories"])


def test_empty_rows_and_single_layer(gc, orc):
    """Outputs without any input (their value is relu(bias)) and a one-layer network."""
    N, B = 64, 20
    print("empty rows", flush=True)
    rng = np.random.default_rng(2)
    nnz = rng.integers(0, 6, size=N)
    nnz[:5] = 0
    csr = sort_rows(random_csr(rng, N, nnz, "general"))
    feats = rng.uniform(0, 5, size=(B, N)).astype(np.float32)
    feats[3] = 0
    for bias in (-0.1, 0.2):
        with gc.Network(N, B, 1, bias=bias) as net:
            net.set_layer_csr(0, *csr)
            net.inspect()
            net.set_features_dense(feats)
            net.run(prune=False, collect_counts=True)
            y, act = orc.layer(feats, csr, bias)
            assert same_floats(net.activations(np.arange(B, dtype=np.int32)), y)
            assert np.array_equal(net.categories(), np.nonzero(act)[0])
            assert net.active_count(0) == int(act.sum())
    # a layer without a single entry between two ordinary ones: every output is relu(bias)
    N2 = 256
    empty = (np.zeros(N2 + 1, np.int32), np.zeros(0, np.int32), np.zeros(0, np.float32))
    layers = [orc.gen_layer_csr(1, 0, N2), empty, sort_rows(random_csr(rng, N2, rng.integers(1, 6, size=N2), "general"))]
    f2 = orc.gen_features(1, N2, 0, B, 0.2, 0.8)
    for bias in (-0.1, 0.2):
        ref = orc.infer(f2, layers, bias, prune=False, keep={2})
        with gc.Network(N2, B, 3, bias=bias) as net:
            for l, c in enumerate(layers):
                net.set_layer_csr(l, *c)
            net.inspect()
            assert net.layer_plan(1).kernel == gc.KERNEL_GATHER and net.layer_plan(2).kernel == gc.KERNEL_TILED
            net.set_features_dense(f2)
            net.run(prune=False, collect_counts=True)
            assert same_floats(net.activations(np.arange(B, dtype=np.int32)), ref["kept"][2][1])
            assert np.array_equal(net.categories(), ref["active_ids"][2])


def test_cli_driver_on_tsv_files(gc, orc, tmp_path):
    """spdnn_network (the reference's `exe neuron batch layer` command line) on challenge-format
    TSV files in the reference's directory layout; categories against the oracle."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(gc.lib_path()), "spdnn_network")
    if not os.path.exists(exe):
        pytest.skip("driver not built")
    N, B, L = 1024, 300, 4
    print("cli driver", flush=True)
    data = tmp_path / "data"
    (data / ("neuron%d" % N)).mkdir(parents=True)
    layers = [orc.gen_layer_csr(6, l, N) for l in range(L)]
    for l, (rowptr, col, val) in enumerate(layers):
        with open(gc.weight_file_name(str(data), N, l), "w") as f:
            f.writelines("%d\t%d\t%.9g\n" % (col[e] + 1, j + 1, val[e]) for j in range(N) for e in range(rowptr[j], rowptr[j + 1]))
    feats = orc.gen_features(6, N, 0, B, 0.10, 0.55)
    with open(data / ("sparse-images-%d.tsv" % N), "w") as f:
        rr, cc = np.nonzero(feats)
        f.writelines("%d\t%d\t1\n" % (r + 1, c + 1) for r, c in zip(rr, cc))
    ref = orc.infer(feats, layers, -0.3, prune=True)
    out = tmp_path / "categories.tsv"
    r = subprocess.run([exe, str(N), str(B), str(L), "--data", str(data), "--categories", str(out)],
                       capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    for l in range(L):
        assert "layer %d, batch = %d" % (l, len(ref["active_ids"][l])) in r.stdout
    got = np.array([int(x) for x in out.read_text().split()], dtype=np.int64)
    assert np.array_equal(got, ref["categories"] + 1)
    # the written file is in the challenge's truth-file format: the driver checks itself against it
    r = subprocess.run([exe, str(N), str(B), str(L), "--data", str(data), "--truth", str(out), "--quiet"],
                       capture_output=True, text=True, timeout=100)
    assert r.returncode == 0 and "Challenge PASSED" in r.stdout
    wrong = tmp_path / "wrong.tsv"
    wrong.write_text("".join("%d\n" % x for x in got[:-1]))
    r = subprocess.run([exe, str(N), str(B), str(L), "--data", str(data), "--truth", str(wrong), "--quiet"],
                       capture_output=True, text=True, timeout=100)
    assert r.returncode == 3 and "Challenge FAILED" in r.stdout
    # without files the driver falls back to the seeded generator
    r = subprocess.run([exe, str(N), "200", "3", "--data", str(tmp_path / "nowhere"), "--quiet"],
                       capture_output=True, text=True, timeout=100)
    assert r.returncode == 0 and "seeded generator" in r.stdout


def test_packed_binary_files(gc, orc, tmp_path):
    """Weights and features in the packed binary layout the reference's library benchmarks read
    (benchmark/cusparse/cusparse.cu:318-383), through the library and through the command-line
    driver; the oracle reads the same files with its own reader."""
    import os
    import subprocess
    N, B, L = 1024, 333, 3
    print("packed binary", flush=True)
    rng = np.random.default_rng(4)
    layers = [orc.gen_layer_csr(12, l, N) for l in range(L)]
    with open(tmp_path / ("neuron%d.bin" % N), "wb") as f:
        for rowptr, col, val in layers:
            row = np.repeat(np.arange(N, dtype=np.int32), np.diff(rowptr))
            perm = rng.permutation(len(col))
            (row[perm] + 1).astype("<i4").tofile(f)
            (col[perm] + 1).astype("<i4").tofile(f)
            val[perm].astype("<f4").tofile(f)
    feats = orc.gen_features(12, N, 0, B + 20, 0.10, 0.55)     # 20 images more than the batch
    img, neu = np.nonzero(feats)
    perm = rng.permutation(len(img))
    with open(tmp_path / ("sparse-images-%d.bin" % N), "wb") as f:
        (neu[perm] + 1).astype("<i4").tofile(f)
        (img[perm] + 1).astype("<i4").tofile(f)
        feats[img[perm], neu[perm]].astype("<f4").tofile(f)
    wpath, fpath = str(tmp_path / ("neuron%d.bin" % N)), str(tmp_path / ("sparse-images-%d.bin" % N))
    ofeats = orc.read_features_bin(fpath, N, B)
    assert np.array_equal(ofeats, feats[:B])
    olayers = [orc.read_weights_bin(wpath, N, l) for l in range(L)]
    ref = orc.infer(ofeats, [(rp, *_sorted_rows(rp, c, v)) for rp, c, v in olayers], -0.3, prune=True)
    with gc.Network(N, B, L, bias=-0.3) as net:
        net.load_layers_bin(wpath)
        net.inspect()
        net.load_features_bin(fpath, B)
        net.run(prune=True, collect_counts=True)
        assert np.array_equal(net.categories(), ref["categories"])
        for l in range(L):
            assert net.active_count(l) == len(ref["active_ids"][l])
        assert np.array_equal(net.activations(ref["categories"][:50].astype(np.int32)), ref["y"][:50])
    exe = os.path.join(os.path.dirname(gc.lib_path()), "spdnn_network")
    if os.path.exists(exe):
        out = tmp_path / "cat.tsv"
        r = subprocess.run([exe, str(N), str(B), str(L), "--data", str(tmp_path), "--categories", str(out), "--quiet"],
                           capture_output=True, text=True, timeout=100)
        assert r.returncode == 0, r.stdout + r.stderr
        got = np.array([int(x) for x in out.read_text().split()], dtype=np.int64)
        assert np.array_equal(got, ref["categories"] + 1)


def _sorted_rows(rowptr, col, val):
    col, val = col.copy(), val.copy()
    for j in range(len(rowptr) - 1):
        a, b = rowptr[j], rowptr[j + 1]
        o = np.argsort(col[a:b], kind="stable")
        col[a:b], val[a:b] = col[a:b][o], val[a:b][o]
    return col, val


def test_handle_lifecycle(gc, orc):
    """Two networks alive at once with interleaved runs, features replaced between runs, a layer
    replaced after a run (inspect again, set features again), and no device memory left behind by
    create/run/destroy cycles."""
    print("lifecycle", flush=True)
    N, B, L = 512, 300, 3
    la = [orc.gen_layer_csr(31, l, N) for l in range(L)]
    lb = [orc.gen_layer_csr(32, l, N, 8) for l in range(L)]
    fa = orc.gen_features(31, N, 0, B, 0.1, 0.6)
    fb = orc.gen_features(32, N, 0, 77, 0.3, 0.9)
    ra = orc.infer(fa, la, -0.3, prune=True)
    rb = orc.infer(fb, lb, -0.05, prune=True)
    with gc.Network(N, B, L, bias=-0.3) as a, gc.Network(N, B, L, bias=-0.05) as b:
        for l in range(L):
            a.set_layer_csr(l, *la[l])
            b.set_layer_csr(l, *lb[l])
        a.inspect()
        b.inspect()
        a.set_features_dense(fa)
        b.set_features_dense(fb)
        a.run(first_layer=0, n_layers=1)
        b.run(first_layer=0, n_layers=2)
        a.run(first_layer=1, n_layers=2)
        b.run(first_layer=2, n_layers=1)
        assert np.array_equal(a.categories(), ra["categories"]) and np.array_equal(b.categories(), rb["categories"])
        # new features on the same handle (smaller batch), then the first ones again
        a.set_features_dense(fb)
        a.run()
        assert np.array_equal(a.categories(), orc.infer(fb, la, -0.3, prune=True)["categories"])
        a.set_features_dense(fa)
        a.run()
        assert np.array_equal(a.categories(), ra["categories"])
        # replace a layer: everything before the next inspect is refused, then results follow the new layer
        a.set_layer_csr(1, *lb[1])
        with pytest.raises(gc.SpdnnError):
            a.run()
        a.inspect()
        with pytest.raises(gc.SpdnnError):
            a.run()                     # features went with the old plans
        a.set_features_dense(fa)
        a.run()
        want = orc.infer(fa, [la[0], lb[1], la[2]], -0.3, prune=True)
        assert np.array_equal(a.categories(), want["categories"])
        k = min(20, len(want["categories"]))
        assert same_floats(a.activations(want["categories"][:k].astype(np.int32)), want["y"][:k])
    free0, total = gc.device_memory()
    assert 0 < free0 <= total
    for _ in range(4):
        with gc.Network(4096, 4096, 2) as net:
            net.synth_layers(1)
            net.inspect()
            net.synth_features(1, 4096, 0.1, 0.6)
            net.run()
    free1, _ = gc.device_memory()
    assert free0 - free1 < (64 << 20), "device memory not returned: %d bytes" % (free0 - free1)


def test_randomized_shapes_and_options(gc, orc, monkeypatch):
    """400 seeded random cases: widths 32 ... 4096 (also not powers of two), batches around the
    row-block sizes, 1-6 layers of every class and weight mode, bias below, at and above zero,
    pruning, fused launches, streamed plans, all row-block sizes - final categories, activations
    and per-layer counts against the oracle, on a first run and on a repeated one."""
    from helpers import hub_block_csr, radix_like_csr
    for case in range(400):
        rng = np.random.default_rng(770000 + case)
        N = int(rng.choice([32, 48, 64, 100, 256, 384, 1000, 1024, 2048, 4096]))
        B = int(rng.choice([1, 3, 63, 64, 65, 255, 257, 700, 1500]))
        L = int(rng.integers(1, 7))
        rl = int(rng.choice([1, 2, 4]))
        bias = float(rng.choice([-0.3, -0.05, 0.0, 0.1]))
        prune = bool(rng.integers(0, 2)) and bias <= 0
        fuse = int(rng.choice([0, 0, 3]))
        window = int(rng.choice([0, 0, 2, 3]))
        minchain = int(rng.choice([256, 4096]))
        values = str(rng.choice(["uniform", "pow2", "general"]))
        # a third of the cases: every layer of one kind and row length, so that consecutive layers can share a
        # persistent launch (switched on and off, queued per XCD or not, with a wait limit of zero now and then)
        same_kind = str(rng.choice(["circ", "radix", "hub", "gather", "radix-common"])) if rng.random() < 0.45 else None
        same_nnz = int(rng.choice([4, 16, 32]))
        persist = dict(SPDNN_PERSIST=str(int(rng.integers(0, 2))), SPDNN_PERSIST_XCD=str(int(rng.choice([-1, 0, 1]))),
                       SPDNN_PERSIST_LIGHT_SYNC=str(int(rng.integers(0, 2))), SPDNN_RESIDENT=str(int(rng.choice([1, 1, 0]))),
                       SPDNN_COMMON_ORDER=str(int(rng.choice([1, 1, 0]))), SPDNN_BAND_RESIDENT=str(int(rng.choice([1, 0]))),
                       SPDNN_BAND_RESIDENT_MIN_LAYERS=str(int(rng.choice([2, 6]))))
        common_perm = rng.permutation(N)
        wait_us = int(rng.choice([0, 0, -1]))
        layers, kinds = [], []
        for l in range(L):
            kind = same_kind or str(rng.choice(["circ", "circ", "gather", "radix", "hub"]))
            if kind in ("radix", "hub", "radix-common") and (N % 32 or N < 64):
                kind = "circ"
            if kind == "circ":
                nnz = same_nnz if same_kind else int(rng.integers(1, 41))
                rp, c, v = orc.gen_layer_csr(int(rng.integers(0, 1000)), l, N, int(min(N, nnz)))
                if values == "pow2":
                    v = np.ldexp(1.0, rng.integers(-6, -2, size=len(v))).astype(np.float32)
                elif values == "general":
                    v = rng.uniform(-0.1, 0.2, size=len(v)).astype(np.float32)
                layers.append((rp, c, v))
            elif kind == "gather":
                layers.append(sort_rows(random_csr(rng, N, rng.integers(0, min(N, 24), size=N), values)))
            elif kind == "radix":
                layers.append(radix_like_csr(rng, N, int(16 * rng.integers(1, N // 16)), values))
            elif kind == "radix-common":   # one hidden numbering for all such layers, strides 16 and 32 mostly
                layers.append(radix_like_csr(rng, N, int(rng.choice([16, 16, 32, 32, 64])) % N or 16, values, perm=common_perm))
            else:
                layers.append(hub_block_csr(rng, N, values))
            kinds.append(kind)
        dens = float(rng.choice([0.05, 0.3, 0.8]))
        feats = (rng.uniform(0, 3, size=(B, N)) * (rng.random((B, N)) < dens)).astype(np.float32)
        what = dict(case=case, N=N, B=B, L=L, rl=rl, bias=bias, prune=prune, fuse=fuse, window=window,
                    minchain=minchain, values=values, kinds=kinds, dens=dens, persist=persist, wait_us=wait_us)
        if case % 50 == 0:
            print("random case", what, flush=True)
        for k, v in persist.items():
            monkeypatch.setenv(k, v)
        monkeypatch.setenv("SPDNN_ROWS_PER_LANE", str(rl))
        monkeypatch.setenv("SPDNN_RUN_CHAINS_MIN_N", str(minchain))
        monkeypatch.setenv("SPDNN_BLOCK_FORM_MAX_ELEMS", str(int(rng.choice([0, 1 << 26]))))   # run chains: band walk or BLOCK form
        monkeypatch.setenv("SPDNN_TILED_MIN_ROWS", str(int(rng.choice([0, 8192]))))            # unstructured layers: tiles or their gather form
        monkeypatch.setenv("SPDNN_ROWTILE", str(int(rng.integers(0, 2))))                      # ... and which of the two forms with LDS staging
        monkeypatch.setenv("SPDNN_STREAM_MIN_BYTES", str(int(rng.choice([0, 96 << 20]))))      # band walk with or without streaming hints
        ref = orc.infer(feats, layers, bias, prune=False, keep={L - 1})
        with gc.Network(N, B, L, bias=bias) as net:
            if window:
                net.set_plan_window(window)
            for l, csr in enumerate(layers):
                net.set_layer_csr(l, *csr)
            net.inspect()
            net.set_features_dense(feats)
            for rep in range(2):
                net.run(prune=prune, collect_counts=True, fuse_layers=fuse, persist_wait_us=wait_us)
                assert np.array_equal(net.categories(), ref["active_ids"][L - 1]), what
                assert same_floats(net.activations(np.arange(B, dtype=np.int32)), ref["kept"][L - 1][1]), what
                if bias <= 0:
                    assert [net.active_count(l) for l in range(L)] == [len(a) for a in ref["active_ids"]], what


def test_randomized_call_sequences(gc, orc, monkeypatch):
    """150 seeded random sequences of calls on one handle - new features of another batch size,
    whole runs (pruned or not, fused, different compaction thresholds), continued partial runs,
    activations of random rows, categories, a replaced layer with a new inspection - followed on
    the side by the oracle, layer by layer."""
    from helpers import hub_block_csr, radix_like_csr

    def make_layer(rng, N, l, values):
        kind = str(rng.choice(["circ", "circ", "gather", "radix", "hub"]))
        if kind == "circ":
            rp, c, v = orc.gen_layer_csr(int(rng.integers(0, 1000)), l, N, int(min(N, rng.integers(2, 41))))
            if values == "pow2":
                v = np.ldexp(1.0, rng.integers(-5, -2, size=len(v))).astype(np.float32)
            elif values == "general":
                v = rng.uniform(-0.05, 0.2, size=len(v)).astype(np.float32)
            return rp, c, v
        if kind == "gather":
            return sort_rows(random_csr(rng, N, rng.integers(0, min(N, 24), size=N), values))
        if kind == "radix":
            return radix_like_csr(rng, N, int(16 * rng.integers(1, N // 16)), values)
        return hub_block_csr(rng, N, values)

    for case in range(150):
        rng = np.random.default_rng(880000 + case)
        N = int(rng.choice([64, 256, 1024, 2048]))
        maxB = int(rng.choice([65, 300, 1100]))
        L = int(rng.integers(2, 9))
        bias = float(rng.choice([-0.3, -0.1, 0.0]))
        values = str(rng.choice(["uniform", "pow2", "general"]))
        window = int(rng.choice([0, 0, 2]))
        monkeypatch.setenv("SPDNN_ROWS_PER_LANE", str(int(rng.choice([1, 2, 4]))))
        monkeypatch.setenv("SPDNN_RUN_CHAINS_MIN_N", str(int(rng.choice([256, 4096]))))
        monkeypatch.setenv("SPDNN_BLOCK_FORM_MAX_ELEMS", str(int(rng.choice([0, 1 << 26]))))
        monkeypatch.setenv("SPDNN_PERSIST_XCD", str(int(rng.choice([-1, 0, 1]))))
        monkeypatch.setenv("SPDNN_PERSIST_LIGHT_SYNC", str(int(rng.integers(0, 2))))
        if rng.random() < 0.4:   # every layer the same band layer: runs of them share persistent launches
            one = make_layer(np.random.default_rng(case), N, 0, values)
            layers = [one for l in range(L)]
        else:
            layers = [make_layer(rng, N, l, values) for l in range(L)]
        what = dict(case=case, N=N, maxB=maxB, L=L, bias=bias, values=values, window=window)
        if case % 25 == 0:
            print("random sequence", what, flush=True)
        log = []
        with gc.Network(N, maxB, L, bias=bias) as net:
            if window:
                net.set_plan_window(window)
            for l, csr in enumerate(layers):
                net.set_layer_csr(l, *csr)
            net.inspect()
            feats, done, y = None, 0, None     # done = layers applied to y so far
            for step in range(int(rng.integers(4, 14))):
                op = str(rng.choice(["feat", "run_all", "run_part", "acts", "cats", "replace", "threshold"]))
                if feats is None:
                    op = "feat"
                log.append(op)
                if op == "feat":
                    B = int(rng.integers(1, maxB + 1))
                    dens = float(rng.choice([0.02, 0.2, 0.7]))
                    feats = (rng.uniform(0, 3, size=(B, N)) * (rng.random((B, N)) < dens)).astype(np.float32)
                    net.set_features_dense(feats)
                    y, done = feats.copy(), 0
                elif op in ("run_all", "threshold"):
                    thr = float(rng.choice([0.0, 0.3, 1.0])) if op == "threshold" else 0.0
                    net.run(prune=bool(rng.integers(0, 2)), collect_counts=True, fuse_layers=int(rng.choice([0, 2, 4])),
                            compact_threshold=thr, persist_wait_us=int(rng.choice([0, 0, 0, -1])))
                    ref = orc.infer(feats, layers, bias, prune=False, keep={L - 1})
                    y, done = ref["kept"][L - 1][1], L
                    assert [net.active_count(l) for l in range(L)] == [len(a) for a in ref["active_ids"]], (what, log)
                elif op == "run_part":
                    if done >= L:
                        y, done = feats.copy(), 0
                    nl = int(rng.integers(1, L - done + 1))
                    net.run(prune=bool(rng.integers(0, 2)), first_layer=done, n_layers=nl, collect_counts=True)
                    for l in range(done, done + nl):
                        y, _ = orc.layer(y, layers[l], bias)
                    done += nl
                elif op == "acts":
                    B = feats.shape[0]
                    rows = rng.permutation(B)[: int(rng.integers(1, B + 1))].astype(np.int32)
                    assert same_floats(net.activations(rows), y[rows]), (what, log)
                elif op == "cats" and done > 0:
                    assert np.array_equal(net.categories(), np.nonzero((y != 0).any(axis=1))[0]), (what, log)
                elif op == "replace":
                    l = int(rng.integers(0, L))
                    layers[l] = make_layer(rng, N, l, values)
                    net.set_layer_csr(l, *layers[l])
                    net.inspect()
                    feats = None


def test_out_of_device_memory(gc, orc):
    """Feature buffers beyond the device's memory: an error code and a message, no abort, and the
    device is usable afterwards."""
    free0, total = gc.device_memory()
    rows = int(total / (65536 * 4) / 2)              # three buffers of this many rows cannot fit
    with gc.Network(65536, rows, 2, bias=-0.45) as net:
        net.synth_layers(0)
        net.inspect()
        with pytest.raises(gc.SpdnnError) as e:
            net.synth_features(0, 1000)
        assert e.value.code == 5 and "memory" in e.value.message
    with gc.Network(1024, 500, 3) as net:
        net.synth_layers(0)
        net.inspect()
        net.synth_features(0, 500)
        assert net.run().layers_run >= 1
    free1, _ = gc.device_memory()
    assert free0 - free1 < (512 << 20)


def test_zero_bias_into_the_denormal_range(gc, orc):
    """Bias 0 and power-of-two weights of 1/16, 8 per row: activations halve (at least) per layer and
    reach the denormal range after ~120 layers, where a product no longer is exact.  The library
    must not take the fused multiply-add shortcut there: bit-equal to the oracle on every layer."""
    N, K, L, B = 256, 8, 140, 64
    print("denormal range", flush=True)
    rng = np.random.default_rng(0)
    layers = []
    for l in range(L):
        rowptr, col, _ = orc.gen_layer_csr(5, l, N, K)
        layers.append((rowptr, col, np.full(len(col), 2.0 ** -4, np.float32)))
    feats = rng.uniform(0.3, 1.0, size=(B, N)).astype(np.float32)
    ref = orc.infer(feats, layers, 0.0, prune=False, keep=set(range(L)))
    assert 0 < ref["kept"][L - 1][1].max() < 1e-40          # the chain does end in denormals
    rows = np.arange(B, dtype=np.int32)
    with gc.Network(N, B, L, bias=0.0) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        assert net.layer_plan(0).kernel == gc.KERNEL_BAND and net.layer_plan(0).exact_products == 1
        net.set_features_dense(feats)
        for l in range(L):
            net.run(prune=False, first_layer=l, n_layers=1)
            if l % 10 == 9 or l > 115:
                assert same_floats(net.activations(rows), ref["kept"][l][1]), "layer %d" % l
        # features so small that even the first product would underflow are refused
        tiny = feats.copy()
        tiny[3, 7] = 1e-35
        with pytest.raises(gc.SpdnnError) as e:
            net.set_features_dense(tiny)
        assert e.value.code == 1 and "2^-100" in e.value.message


def test_reference_side_binding(gc, orc, tmp_path):
    """oracle/_ref/ref_binding is the binding a maintainer of the reference would add to its
    driver, compiled against the reference's own host code: the reference's COOMatrix loads and
    sorts the weight files, the features are read as its read_input does, the rest goes through
    the C ABI.  Built only where the reference is mounted; the prebuilt program travels."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "oracle", "_ref", "ref_binding")
    if not os.path.exists(exe):
        pytest.skip("oracle/_ref/ref_binding not built (reference not mounted at build time)")
    N, B, L = 1024, 200, 3
    print("reference-side binding", flush=True)
    data = tmp_path / "data"
    (data / ("neuron%d" % N)).mkdir(parents=True)
    rng = np.random.default_rng(8)
    layers = [orc.gen_layer_csr(14, l, N) for l in range(L)]
    for l, (rowptr, col, val) in enumerate(layers):
        lines = ["%d\t%d\t%.9g\n" % (col[e] + 1, j + 1, val[e]) for j in range(N) for e in range(rowptr[j], rowptr[j + 1])]
        rng.shuffle(lines)
        with open(gc.weight_file_name(str(data), N, l), "w") as f:
            f.writelines(lines)
    feats = orc.gen_features(14, N, 0, B, 0.10, 0.55)
    with open(data / ("sparse-images-%d.tsv" % N), "w") as f:
        rr, cc = np.nonzero(feats)
        f.writelines("%d\t%d\t1\n" % (r + 1, c + 1) for r, c in zip(rr, cc))
    ref = orc.infer(feats, layers, -0.3, prune=True)
    r = subprocess.run([exe, str(N), str(B), str(L), str(data), "-0.3"], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    for l in range(L):
        assert "layer %d, batch = %d" % (l, len(ref["active_ids"][l])) in r.stdout
    got = np.array([int(x.split()[1]) for x in r.stdout.splitlines() if x.startswith("category ")], dtype=np.int64)
    assert np.array_equal(got, ref["categories"])
