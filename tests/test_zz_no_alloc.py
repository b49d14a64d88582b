"""The entry point that allocates nothing (spdnn_get_activations_noalloc) against the entry point
it is a variant of (spdnn_get_activations), through the C ABI, bit for bit."""
import numpy as np
import pytest

from helpers import same_floats

pytestmark = pytest.mark.gpu


def test_activations_without_allocation(gc, orc):
    N, L = 1024, 10
    layers = [orc.gen_layer_csr(9, l, N) for l in range(L)]
    with gc.Network(N, 1500, L, bias=-0.3) as net:
        for l, csr in enumerate(layers):
            net.set_layer_csr(l, *csr)
        net.inspect()
        rng = np.random.default_rng(12)
        # first call: 1500 rows, pruned run with repacks (the row table matters), 700 rows asked for in random
        # order, dead rows among them; second call right after it: a smaller batch and fewer rows
        for B, nreq in ((1500, 700), (300, 100)):
            print("no-alloc activations: batch %d, %d rows" % (B, nreq), flush=True)
            feats = orc.gen_features(21 + B, N, 0, B, 0.10, 0.50)
            net.set_features_dense(feats)
            r = net.run(prune=True, collect_counts=True)
            ref = orc.infer(feats, layers, -0.3, prune=False, keep={L - 1})
            rows = rng.permutation(B)[:nreq].astype(np.int32)
            calls0 = gc.device_alloc_calls()
            got = net.activations_noalloc(rows)
            assert gc.device_alloc_calls() == calls0          # the library allocated nothing during the call ...
            want = net.activations(rows)
            assert gc.device_alloc_calls() > calls0           # ... which the counter would have seen
            assert same_floats(got, want)
            assert same_floats(got, ref["kept"][L - 1][1][rows])
            assert got.any() and not got.all(axis=1).all()        # survivors and dead rows both present
            if B == 1500:
                assert r.compactions >= 1
        # before any layer has run: the features themselves
        net.set_features_dense(feats)
        assert same_floats(net.activations_noalloc(rows), feats[rows])
        with pytest.raises(gc.SpdnnError) as e:
            net.activations_noalloc(np.array([B], np.int32))
        assert e.value.code == 1
