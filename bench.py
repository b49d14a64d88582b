#!/usr/bin/env python3
"""Benchmark of the Sparse DNN inference hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cfg4] [--layers L]

A step is one pass of the whole layer chain over the full batch (the headline configuration:
N=65536, 1920 layers, batch 60000, bias -0.45, seed 0, synthetic weights and features generated
by the library's seeded generator).  Reported on ONE JSON line:

  value        edges/s = batch * N * 32 * layers / t of the SUSTAINED run: pruning off, every
               layer processes the full batch, nothing skipped (with the literal inputs every row
               dies within two layers, so the pruned run would be timing empty layers).
  roofline     band-walk kernel: algorithmic bytes per launch (8*B*N + 8*nnz + 4*(N+1)) over the
               average launch duration measured with HIP events on the library's stream, against
               the 8 TB/s HBM peak.
  cpu_baseline the CPU oracle (oracle/) timed on this box's host cores on a bounded sample of the
               same workload (the first layers, chained, on the first rows).
  literal      the run as configured (pruning on): edges/s as defined, layers actually launched,
               per-layer active rows; and the parity gate of a row sample against the oracle.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

CONFIGS = {
    # name: (neuron, layers, batch, bias)
    "cfg0": (1024, 120, 6000, -0.30),
    "cfg1": (1024, 120, 60000, -0.30),
    "cfg2": (4096, 480, 60000, -0.35),
    "cfg3": (16384, 1920, 60000, -0.40),
    "cfg4": (65536, 1920, 60000, -0.45),
}
HBM_PEAK_GBPS = 8000.0
METRIC = "inference edges/sec at N=65536×1920 layers, batch 60000; % HBM roofline"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def radix_layer(rng, n, stride, perm=None):
    """A layer with the structure of the challenge's RadiX-Net files: the 16 outputs of group g read the
    two 16-wide input runs [16g, 16g+16) and [16g+stride, 16g+stride+16) (mod n), hidden behind random
    relabellings of inputs and outputs (perm: behind that one relabelling for both, the network's common
    neuron numbering); 32 entries of 1/16 per row.  CSR with row = output neuron."""
    pin, pout = (perm, perm) if perm is not None else (rng.permutation(n).astype(np.int32), rng.permutation(n))
    base = (np.arange(n) // 16 * 16)[:, None]
    run = np.arange(16)[None, :]
    ins = np.concatenate([base + run, (base + stride + run) % n], axis=1)
    col = np.empty((n, 32), np.int32)
    col[pout] = np.sort(pin[ins], axis=1)
    return (np.arange(n + 1, dtype=np.int32) * 32, col.reshape(-1), np.full(n * 32, 0.0625, np.float32))


def common_band_layer(perm):
    """A convolution-like layer over the neuron order `perm` (common to all layers): the neuron at place t
    reads the neurons at places t-31 .. t; 32 entries of 1/16 per row.  Consecutive layers of this kind write
    their outputs where the next one's band reads them, so the library runs them two per launch."""
    n = len(perm)
    col = np.empty((n, 32), np.int32)
    col[perm] = np.sort(perm[(np.arange(n)[:, None] - np.arange(32)[None, :]) % n], axis=1)
    return (np.arange(n + 1, dtype=np.int32) * 32, col.reshape(-1), np.full(n * 32, 0.0625, np.float32))


def irregular_layer(rng, n, kmax=24):
    """A layer without structure: every output reads 1..kmax random inputs with random weights."""
    lens = rng.integers(1, kmax + 1, size=n)
    rowptr = np.zeros(n + 1, np.int32)
    np.cumsum(lens, out=rowptr[1:])
    order = np.argsort(rng.random((n, n), dtype=np.float32), axis=1)[:, :kmax].astype(np.int32)
    col = np.concatenate([np.sort(order[j, :lens[j]]) for j in range(n)]).astype(np.int32)
    val = rng.uniform(0.02, 0.12, size=len(col)).astype(np.float32)
    return rowptr, col, val


def cpu_literal_run(orc, layer_csr, N, L, B, bias, seed, dens_hi, chunk=4096):
    """The literal run of a configuration on the CPU oracle (pruning on, every row of the batch, all cores), in row
    chunks to bound the memory: seconds and the per-layer active-row counts."""
    t_lit = 0.0
    counts = np.zeros(L, np.int64)
    layers_cache = {}
    for r0 in range(0, B, chunk):
        y = orc.gen_features(seed, N, r0, min(chunk, B - r0), 0.10, dens_hi)
        gid = np.arange(len(y), dtype=np.int32)
        for l in range(L):
            if l not in layers_cache:
                layers_cache[l] = layer_csr(l)
            t0 = time.perf_counter()
            y, act = orc.layer(y, layers_cache[l], bias)
            y, gid = orc.compact(y, act, gid)
            t_lit += time.perf_counter() - t0
            counts[l] += len(gid)
            if len(gid) == 0:
                break
    return t_lit, counts


def sustained_block(gc, name, seed, log, per_layer_too, with_cpu=True):
    """One BASELINE configuration other than the headline one, sustained (pruning off, full batch at every layer): ms per
    layer and fraction of the HBM roofline on the configured features (all-zero activations from layer 2 on) and on live
    data (densities up to 0.7: rows survive every layer), two timed passes each after one warm-up pass; for the narrow
    configurations also with every layer as its own launch (the default shares resident or persistent launches where it pays)."""
    N, L, B, bias = CONFIGS[name]
    t0 = time.time()
    net = gc.Network(N, B, L, bias=bias)
    net.synth_layers(seed)
    net.inspect()
    alg = 8.0 * B * N + 8.0 * 32 * N + 4.0 * (N + 1)
    out = {"neuron": N, "layers": L, "batch": B, "alg_bytes_per_layer": alg}

    def timed(fuse):
        net.run(prune=False, fuse_layers=fuse)
        best, r = None, None
        for _ in range(2):
            r = net.run(prune=False, fuse_layers=fuse)
            best = r.ms_total if best is None else min(best, r.ms_total)
        ms = best / L
        return {"ms_per_layer": ms, "frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "launches_per_pass": int(r.launches),
                "persistent_launches_per_pass": int(r.persistent_launches), "persistent_fallbacks": int(r.persistent_fallbacks),
                "resident_launches_per_pass": int(r.resident_launches), "rows_nonzero_at_end": int(r.active_rows)}

    net.synth_features(seed, B, 0.10, 0.25)
    out["zeros"] = timed(0)
    if out["zeros"]["resident_launches_per_pass"]:
        out["zeros"]["frac"] = None
        out["zeros"]["note"] = ("resident launches: a workgroup whose 16 rows are all zero leaves at once, so this figure is no "
                                "measure of the kernels - the live figures are")
    net.synth_features(seed, B, 0.10, 0.70)
    out["live"] = timed(0)
    if per_layer_too:
        out["live_one_launch_per_layer"] = timed(1)
    lit = net.run(prune=True, collect_counts=True)
    out["literal_live_pruned_ms"] = lit.ms_total
    # the literal run of the configuration as BASELINE defines it (densities up to 0.25, pruning on), GPU and CPU side by side
    net.synth_features(seed, B, 0.10, 0.25)
    lit = net.run(prune=True, collect_counts=True)
    gpu_counts = [int(net.active_count(l)) for l in range(min(L, 8))]
    out["literal"] = {"gpu_ms": lit.ms_total, "active_rows_first_layers": gpu_counts, "categories": int(lit.active_rows)}
    if with_cpu:
        from oracle import oracle as orc
        t_cpu, cpu_counts = cpu_literal_run(orc, lambda l: orc.gen_layer_csr(seed, l, N), N, L, B, bias, seed, 0.25)
        out["literal"].update({"cpu_s": t_cpu, "cpu_cores": orc.get_threads(),
                               "counts_equal": [int(c) for c in cpu_counts[:len(gpu_counts)]] == gpu_counts})
    out["band_tuning_rowblocks_shape_seglen"] = net.band_tuning()
    out["feature_buffers_region_paired_candidates_peak_bytes"] = list(net.feature_placement())
    net.close()
    out["wall_s"] = time.time() - t0
    log("other config %s: zeros %.4f ms/layer (frac %s), live %.4f ms/layer (frac %.3f), %.1f s"
        % (name, out["zeros"]["ms_per_layer"], "%.3f" % out["zeros"]["frac"] if out["zeros"]["frac"] is not None else "-",
           out["live"]["ms_per_layer"], out["live"]["frac"], out["wall_s"]))
    return out


def structure_block(gc, structure, N, L, B, bias, log):
    """The other layer classes at a BASELINE shape, sustained on live data (feature densities U[0.10, 0.70], pruning off,
    two timed passes after a warm-up): RadiX-Net-like layers (BLOCK class: strides 16 .. N/2 in turn behind random
    relabellings, 32 nnz/row of 0.0625) or layers without structure (TILED class: 1..24 random inputs per output, random
    weights; bias +0.01 so that rows stay alive), left to the library and with one launch per layer."""
    rng = np.random.default_rng(N)
    t0 = time.time()
    if structure == "radix":
        kinds = [radix_layer(rng, N, 16 << k) for k in range(int(np.log2(N // 16)))]
    else:
        kinds = [irregular_layer(rng, N) for _ in range(4)]
        bias = 0.01
    net = gc.Network(N, B, L, bias=bias)
    for l in range(L):
        net.set_layer_csr(l, *kinds[l % len(kinds)])
    net.inspect()
    net.synth_features(1, B, 0.10, 0.70)
    alg = 8.0 * B * N
    out = {"structure": structure, "neuron": N, "layers": L, "batch": B, "bias": bias,
           "kernel_classes": sorted({int(net.layer_plan(l).kernel) for l in range(L)})}
    for key, fuse in (("default", 0), ("one_launch_per_layer", 1)):
        net.run(prune=False, fuse_layers=fuse)
        best, r = None, None
        for _ in range(2):
            r = net.run(prune=False, fuse_layers=fuse)
            best = r.ms_total if best is None else min(best, r.ms_total)
        ms = best / L
        out[key] = {"ms_per_layer": ms, "algorithmic_bytes_over_time_frac": alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                    "launches_per_pass": int(r.launches), "resident_launches_per_pass": int(r.resident_launches),
                    "rows_nonzero_at_end": int(r.active_rows)}
    net.close()
    out["wall_s"] = time.time() - t0
    log("structure %s N=%d: default %.4f ms/layer, one launch per layer %.4f ms/layer, %.1f s"
        % (structure, N, out["default"]["ms_per_layer"], out["one_launch_per_layer"]["ms_per_layer"], out["wall_s"]))
    return out


def challenge_like_block(gc, N, L, B, bias, log):
    """A run shaped like the challenge's own (the official files are not available offline): RadiX-Net-like layers of
    strides 16, 32, ... N/2 in turn behind random relabellings, batch B of which 3 % are dense rows that survive every
    layer and the rest dies within two layers, pruning on: the whole run's milliseconds."""
    rng = np.random.default_rng(N)
    t0 = time.time()
    kinds = [radix_layer(rng, N, 16 << k) for k in range(int(np.log2(N // 16)))]
    net = gc.Network(N, B, L, bias=bias)
    for l in range(L):
        net.set_layer_csr(l, *kinds[l % len(kinds)])
    net.inspect()
    t_inspect = time.time() - t0
    blk = 3000
    dens = np.where(rng.random(blk) < 0.03, 0.7, 0.05).astype(np.float32)
    part = (rng.random((blk, N), dtype=np.float32) < dens[:, None]).astype(np.float32)
    feats = np.tile(part, (B // blk, 1))
    del part
    net.set_features_dense(feats)
    del feats
    best, r = None, None
    for _ in range(3):
        r = net.run(prune=True, collect_counts=True)
        best = r.ms_total if best is None else min(best, r.ms_total)
    counts = [int(net.active_count(l)) for l in (0, 1, 2, L - 1)]
    plans = sorted({net.layer_plan(l).kernel for l in range(0, L, max(1, L // 16))})
    net.close()
    out = {"neuron": N, "layers": L, "batch": B, "ms": best, "edges_per_s": float(B) * 32.0 * N * L / (best * 1e-3),
           "us_per_layer": best * 1e3 / L, "compactions": int(r.compactions), "carried_rows_at_end": int(r.carried_rows),
           "active_rows_after_layers_0_1_2_last": counts, "launches": int(r.launches),
           "persistent_launches": int(r.persistent_launches), "resident_launches": int(r.resident_launches),
           "kernel_classes": plans, "setup_s": time.time() - t0,
           "inspect_s": t_inspect}
    log("challenge-like N=%d x %d layers: %.3f ms, %d rows at the end, setup %.1f s" % (N, L, best, counts[-1], out["setup_s"]))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--config", default="cfg4", choices=sorted(CONFIGS))
    ap.add_argument("--layers", type=int, default=0, help="override the layer count (quick runs)")
    ap.add_argument("--batch", type=int, default=0, help="override the batch (quick runs)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--fuse", type=int, default=0, help="spdnn_run_options.fuse_layers for the timed runs (1 = no fused launches)")
    ap.add_argument("--structure", default="circulant", choices=["circulant", "radix", "radix-common", "irregular", "common-band"],
                    help="layers: the seeded permuted-stride generator (default, the configured workload), RadiX-Net-like "
                         "layers (one per stride 16, 32, ... n/2, repeated; radix-common: all of them behind one hidden "
                         "neuron numbering, as the layer files of one challenge network), bands over one common order, "
                         "or layers without structure (n <= 4096)")
    ap.add_argument("--density-hi", type=float, default=0.25,
                    help="features: every row's density is drawn from U[0.10, this] (0.25 = the configured workload, whose rows "
                         "all die within two layers; 0.7 = live data: rows survive every layer)")
    ap.add_argument("--cpu-rows", type=int, default=0, help="rows of the CPU sample (0 = auto)")
    ap.add_argument("--cpu-layers", type=int, default=6, help="layers the CPU baseline is timed on")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and the parity gate")
    ap.add_argument("--no-live", action="store_true", help="skip the sustained pass on live data")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the blocks beside the headline run: the other BASELINE configurations, the challenge-like "
                         "pruned runs and the CPU's literal run of the headline configuration")
    ap.add_argument("--survivor-check", type=int, default=0, metavar="ROWS",
                    help="extra (slow): features with densities up to 0.7 so that rows survive every layer; "
                         "the category set of the first ROWS rows after ALL layers is compared with the oracle")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py: this build runs on one GPU (rows never interact, so more GPUs would each take a slice "
            "of the batch with replicated weights; that is not built); run with --gpus 1")
        return 2

    import graphchallenge21_amd as gc

    N, L, B, bias = CONFIGS[args.config]
    if args.layers:
        L = args.layers
    if args.batch:
        B = args.batch
    seed = args.seed
    dev_name, n_cu, hbm = gc.device_info()
    log("device:", dev_name, "CUs", n_cu, "HBM GiB %.0f" % (hbm / 2**30))

    t0 = time.time()
    net = gc.Network(N, B, L, bias=bias)
    kinds = None   # the distinct layers of a structure other than the generator's, used in turn
    if args.structure == "circulant":
        net.synth_layers(seed)

        def layer_csr(l):   # for the CPU legs only: the oracle's own generator (the library generates on its side)
            from oracle import oracle as orc
            return orc.gen_layer_csr(seed, l, N)
    else:
        rng = np.random.default_rng(seed)
        if args.structure == "radix":
            kinds = [radix_layer(rng, N, 16 << k) for k in range(max(1, int(np.log2(N // 16))))]
        elif args.structure == "radix-common":
            perm = rng.permutation(N).astype(np.int32)
            kinds = [radix_layer(rng, N, 16 << k, perm) for k in range(max(1, int(np.log2(N // 16))))]
        elif args.structure == "common-band":
            kinds = [common_band_layer(rng.permutation(N).astype(np.int32))]
        else:
            if N > 4096:
                log("bench.py: --structure irregular is for n <= 4096")
                return 2
            kinds = [irregular_layer(rng, N) for _ in range(4)]
        layer_csr = lambda l: kinds[l % len(kinds)]
        for l in range(L):
            net.set_layer_csr(l, *layer_csr(l))
    net.inspect()
    t_inspect = time.time() - t0
    plans = [net.layer_plan(l) for l in range(L)]
    n_band = sum(1 for p in plans if p.kernel == gc.KERNEL_BAND)
    kernel_names = {gc.KERNEL_BAND: "band_walk_kernel", gc.KERNEL_BLOCK: "block_kernel", gc.KERNEL_GATHER: "gather_kernel",
                    gc.KERNEL_TILED: "tiled_kernel"}
    kernels_used = sorted({kernel_names[p.kernel] for p in plans})
    nnz_layer = float(sum(p.nnz for p in plans)) / L     # the same for every layer except with --structure irregular
    t0 = time.time()
    net.synth_features(seed, B, 0.10, args.density_hi)
    t_features = time.time() - t0
    log("setup: inspector %.1f s (%d/%d layers BAND, kernels %s), plan upload + features %.1f s"
        % (t_inspect, n_band, L, "+".join(kernels_used), t_features))

    # ---- sustained run: the timed steps ---------------------------------------------------
    for i in range(args.warmup):
        r = net.run(prune=False, time_layers=True, fuse_layers=args.fuse)
        log("warmup %d/%d: %.0f ms" % (i + 1, args.warmup, r.ms_total))
    gc.load_library().spdnn_device_synchronize()
    layer_ms = []
    t0 = time.perf_counter()
    ms_events = 0.0
    for i in range(args.steps):
        r = net.run(prune=False, time_layers=True, fuse_layers=args.fuse)
        ms_events += r.ms_total
        layer_ms.append(net.layer_times().copy())
        log("step %d/%d: %.0f ms" % (i + 1, args.steps, r.ms_total))   # between steps, the GPU idle: a progress line
    gc.load_library().spdnn_device_synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = wall_ms / args.steps
    edges = float(B) * float(nnz_layer) * L
    value = edges / (ms_per_step * 1e-3)
    layer_ms = np.concatenate(layer_ms)
    avg_launch_ms = float(layer_ms.mean())
    alg_bytes_launch = 8.0 * B * N + 8.0 * nnz_layer + 4.0 * (N + 1)
    achieved = alg_bytes_launch / (avg_launch_ms * 1e-3) / 1e9
    sustained_final_active = int(r.active_rows)

    # ---- layer 0 alone (live data), and the literal run -------------------------------------
    r0 = net.run(prune=False, first_layer=0, n_layers=1, time_layers=True)
    layer0_ms = float(net.layer_times()[0])
    lit = net.run(prune=True, collect_counts=True)
    lit_counts = []
    for l in range(min(L, 8)):
        lit_counts.append(int(net.active_count(l)))
    lit_categories = int(lit.active_rows)

    # ---- measured copy bandwidth --------------------------------------------------------------
    copy_gbps = gc.measure_copy_bandwidth(1 << 32, 5)          # two plain 4 GiB allocations
    try:
        buffer_copy_gbps = net.buffer_copy_bandwidth(3)            # the work buffers where they lie
    except gc.SpdnnError:
        buffer_copy_gbps = None
    net.synth_features(seed, B, 0.10, args.density_hi)                    # the probe resets the state

    # ---- live data: the same sustained run on features whose rows survive (densities up to 0.7) --
    live = None
    if not args.no_live:
        net.synth_features(seed, B, 0.10, 0.70)
        net.run(prune=False, time_layers=True, n_layers=min(L, 40), fuse_layers=args.fuse)
        rl = net.run(prune=False, time_layers=True, fuse_layers=args.fuse)
        lms = net.layer_times().copy()
        live_ms = float(lms.mean())
        live = {"workload": "same layers, features of density U[0.10,0.70] (rows survive every layer), pruning off, one pass",
                "avg_launch_ms": live_ms, "achieved": alg_bytes_launch / (live_ms * 1e-3) / 1e9,
                "frac": alg_bytes_launch / (live_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, "unit": "GB/s",
                "launches_timed": int(lms.size), "rows_nonzero_at_end": int(rl.active_rows),
                "edges_per_s": edges / (rl.ms_total * 1e-3)}
        net.synth_features(seed, B, 0.10, args.density_hi)

    # ---- CPU baseline + parity gate on a row sample ---------------------------------------------
    cpu = None
    parity = None
    if not args.no_cpu:
        from oracle import oracle as orc
        cores = orc.get_threads()
        rows = args.cpu_rows or max(256, min(B, int(7.0e10 * max(cores, 1) / 16 / (N * 32.0))) // 256 * 256)
        rows = min(rows, B)
        feats = orc.gen_features(seed, N, 0, rows, 0.10, args.density_hi)
        # timed: the first layers of the same workload, chained, on the sample rows (every row kept,
        # as in the sustained run); the first three of them are the parity reference below
        n_cpu = min(L, args.cpu_layers)
        n_check = min(L, 3)
        ref_ids, ref_y = [], []
        y, gid = feats, np.arange(rows, dtype=np.int32)
        t_cpu = 0.0
        for l in range(max(n_cpu, n_check)):
            csr = layer_csr(l)
            t0 = time.perf_counter()
            yo, act = orc.layer(y, csr, bias)
            if l < n_cpu:
                t_cpu += time.perf_counter() - t0
            if l < n_check:
                ref_ids.append(gid[act != 0].copy())
                ref_y.append((gid.copy(), yo))
            y = yo
        cpu = {"value": rows * float(nnz_layer) * n_cpu / t_cpu, "unit": "edges/s", "cores": cores, "kind": "port",
               "sample": "layers 0..%d of the same workload on rows 0..%d, every row kept (%.1f s)"
                         % (n_cpu - 1, rows - 1, t_cpu)}
        # one thread (the reference's CPU checker is single-threaded): layer 0 on a sixteenth of the sample
        r1 = max(64, rows // 16)
        orc.set_threads(1)
        t0 = time.perf_counter()
        orc.layer(feats[:r1], layer_csr(0), bias)
        t1 = time.perf_counter() - t0
        orc.set_threads(cores)
        cpu["single_thread"] = {"value": r1 * float(nnz_layer) / t1, "unit": "edges/s", "cores": 1,
                                "sample": "layer 0 on rows 0..%d (%.1f s)" % (r1 - 1, t1)}
        if args.structure == "circulant":
            # the reference's own CPU-runnable configuration in full: N=1024, 120 layers, batch 6000
            n0, l0, b0, bias0 = CONFIGS["cfg0"]
            lay0 = [orc.gen_layer_csr(seed, l, n0) for l in range(l0)]
            f0 = orc.gen_features(seed, n0, 0, b0, 0.10, 0.25)
            t0 = time.perf_counter()
            res_p = orc.infer(f0, lay0, bias0, prune=True)
            tp = time.perf_counter() - t0
            t0 = time.perf_counter()
            orc.infer(f0, lay0, bias0, prune=False)
            tu = time.perf_counter() - t0
            e0 = float(b0) * n0 * 32 * l0
            cpu["cfg0_full"] = {"cores": cores, "edges": e0, "pruned_s": tp, "pruned_edges_per_s": e0 / tp,
                                "unpruned_s": tu, "unpruned_edges_per_s": e0 / tu,
                                "categories": int(len(res_p["active_ids"][-1]))}
            if not args.no_extras:
                # the literal run of THIS configuration on the CPU (pruning on, every row of the batch, all cores), in row
                # chunks to bound the memory: the run the GPU's `literal` block makes, its per-layer counts compared
                chunk = 4096
                t_lit, cpu_counts = cpu_literal_run(orc, layer_csr, N, L, B, bias, seed, args.density_hi, chunk)
                ran = int(np.count_nonzero(cpu_counts)) + 1
                cpu["literal"] = {"workload": "%s literal: pruning on, batch %d, all %d layers (rows of chunk after chunk of %d)"
                                              % (args.config, B, L, chunk),
                                  "cores": cores, "seconds": t_lit, "edges_per_s": edges / t_lit,
                                  "layers_with_work": min(ran, L), "active_rows_first_layers": [int(c) for c in cpu_counts[:8]],
                                  "categories": int(cpu_counts[L - 1]),
                                  "counts_equal_gpu": [int(c) for c in cpu_counts[:len(lit_counts)]] == lit_counts}
                cpu["literal_%s" % args.config] = cpu["literal"]    # (the same block under the configuration's name)
        ok_ids, ok_y, max_abs = True, True, 0.0
        sample = np.arange(rows, dtype=np.int32)
        for l in range(n_check):
            net.run(prune=True, first_layer=l, n_layers=1, collect_counts=True)
            cats = net.categories()
            ok_ids &= bool(np.array_equal(cats[cats < rows], ref_ids[l]))
            for c0 in range(0, rows, 2048):   # the whole sample, a chunk of rows at a time
                got = net.activations(sample[c0:c0 + 2048])
                want = ref_y[l][1][c0:c0 + 2048]
                ok_y &= bool(np.array_equal(got, want))
                max_abs = max(max_abs, float(np.abs(got - want).max()))
        parity = {"rows": int(rows), "layers": n_check, "active_ids_equal": ok_ids,
                  "activations_bit_equal": ok_y, "max_abs_diff": max_abs}

    survivor = None
    if args.survivor_check > 0:
        from oracle import oracle as orc
        S = min(args.survivor_check, B)
        net.synth_features(seed, B, 0.10, 0.70)
        t0 = time.perf_counter()
        rs = net.run(prune=True, collect_counts=True)
        gpu_s = time.perf_counter() - t0
        cats = net.categories()
        got_y = net.activations(cats[cats < S][:64].astype(np.int32))
        y = orc.gen_features(seed, N, 0, S, 0.10, 0.70)
        gid = np.arange(S, dtype=np.int32)
        t0 = time.perf_counter()
        for l in range(L):
            y, act = orc.layer(y, layer_csr(l), bias)
            y, gid = orc.compact(y, act, gid)
            if l % 200 == 0:
                log("survivor check: oracle layer %d, %d rows alive" % (l, len(gid)))
        survivor = {"rows_checked": int(S), "layers": L, "gpu_categories_total": int(len(cats)),
                    "oracle_categories_in_sample": int(len(gid)),
                    "categories_equal": bool(np.array_equal(cats[cats < S], gid)),
                    "activations_bit_equal": bool(np.array_equal(got_y, y[:64])),
                    "gpu_pruned_run_s": gpu_s, "gpu_compactions": int(rs.compactions), "oracle_s": time.perf_counter() - t0}

    traffic, traffic_source = None, None
    tpath = os.path.join(ROOT, "profiles", "band_walk_cfg4_hbm_traffic.txt")
    if os.path.exists(tpath) and args.config == "cfg4" and B == 60000 and args.structure == "circulant":
        for line in open(tpath):
            if line.startswith("hbm_bytes_per_launch"):
                traffic = float(line.split("=")[1])
                traffic_source = ("profiles/band_walk_cfg4_hbm_traffic.txt: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this "
                                  "command, kept as text; not measured by this process")

    band_tuning = net.band_tuning()
    placement = list(net.feature_placement())
    plan_memory = list(net.plan_memory())
    net.close()

    # ---- beside the headline run: the other BASELINE configurations and challenge-like pruned runs -----------
    other, challenge, structures = None, None, None
    if not args.no_extras and args.structure == "circulant":
        structures = [structure_block(gc, st_, n_, l_, 60000, b_, log)
                      for st_, n_, l_, b_ in (("radix", 1024, 120, -0.30), ("radix", 4096, 128, -0.35), ("irregular", 1024, 64, 0.01),
                                              ("irregular", 4096, 16, 0.01))]
        other = {name: sustained_block(gc, name, seed, log, per_layer_too=name in ("cfg0", "cfg1", "cfg2"), with_cpu=not args.no_cpu)
                 for name in ("cfg0", "cfg1", "cfg2", "cfg3") if name != args.config}
        challenge = {"workload": "RadiX-Net-like layers (strides 16 .. N/2 in turn, random relabellings), batch 60000 with 3 % "
                                 "dense rows that survive, pruning on, whole run; best of three",
                     "runs": [challenge_like_block(gc, n_, l_, 60000, b_, log)
                              for n_, l_, b_ in ((1024, 120, -0.30), (4096, 480, -0.35), (16384, 1920, -0.40), (65536, 1920, -0.45))]}

    out = {
        "metric": METRIC,
        "value": value,
        "unit": "edges/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "%s sustained: N=%d, %d layers%s, batch %d, bias %g, %s, "
                        "pruning off (every layer at full batch), seed %d"
                        % (args.config, N, L, "" if args.structure == "circulant" else " (%s)" % args.structure, B, bias,
                           "32 nnz/row of 0.0625" if args.structure != "irregular" else "1..24 nnz/row, random weights", seed),
            "neuron": N, "layers": L, "batch": B, "bias": bias, "seed": seed,
            "kernel": "band_walk (rows per lane 4, LDS ring, one v_add_f32 per input under one power-of-two weight)" if n_band == L else "+".join(kernels_used),
            "band_tuning_rowblocks_shape_seglen": band_tuning,
            "feature_buffers_region_paired_candidates_peak_bytes": placement,
            "feature_buffers_region_paired_candidates": placement[:2],
            "plan_window_device_bytes_pinned_bytes": plan_memory,
            "final_active_rows": sustained_final_active,
            "launches_per_pass": int(r.launches), "fused_pairs_per_pass": int(r.fused_pairs),
            "persistent_launches_per_pass": int(r.persistent_launches),
            "resident_launches_per_pass": int(r.resident_launches),
            "feature_density": [0.10, args.density_hi],
        },
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": "+".join(kernels_used), "alg_bytes_per_launch": alg_bytes_launch,
                     "avg_launch_ms": avg_launch_ms, "launches_timed": int(layer_ms.size),
                     "note": ("resident launches: the rows stay in LDS between the layers of a launch, so the algorithmic bytes of a "
                              "layer never reach HBM and `frac` (algorithmic bytes over time, against the HBM peak) is not a bound "
                              "here - the kernel is bound by LDS and the vector ALUs"
                              + ("; on the all-zero activations of this run a workgroup leaves the launch as soon as its rows are zero, so "
                                 "`value` is no measure of the kernels either: run with --density-hi 0.7" if args.density_hi <= 0.25 else ""))
                     if r.resident_launches else None,
                     "data": ("all-zero activations from layer 2 on (bias -0.45 kills every row of the configured features); "
                              "see roofline_live for the same run on live data") if args.density_hi <= 0.25 else
                             "live data: feature densities U[0.10, %g]" % args.density_hi,
                     "copy_kernel_gbps_plain_allocations": copy_gbps,
                     "copy_kernel_gbps_work_buffers": buffer_copy_gbps,
                     "frac_of_work_buffer_copy": achieved / buffer_copy_gbps if buffer_copy_gbps else None,
                     # (the names these two had before)
                     "measured_copy_peak_gbps": copy_gbps,
                     "frac_of_measured_copy": achieved / copy_gbps if copy_gbps else None},
        "roofline_live": live,
        "cpu_baseline": cpu,
        "literal": {"workload": "same inputs, pruning on", "edges_per_s": edges / (lit.ms_total * 1e-3),
                    "ms": lit.ms_total, "layers_launched": int(lit.layers_run), "compactions": int(lit.compactions),
                    "active_rows_first_layers": lit_counts, "categories": lit_categories},
        "layer0": {"ms": layer0_ms, "achieved_gbps": alg_bytes_launch / (layer0_ms * 1e-3) / 1e9,
                   "edges_per_s": B * float(nnz_layer) / (layer0_ms * 1e-3)},
        "parity": parity,
        "survivor_check": survivor,
        "setup_s": {"inspector": t_inspect, "upload_and_features": t_features},
        "events_ms_per_step": ms_events / args.steps,
        "other_configs": other,
        "challenge_like": challenge,
        "other_structures": structures,
    }
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
