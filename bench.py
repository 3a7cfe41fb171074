#!/usr/bin/env python3
"""Benchmark of the sparse-convolution hot path on one MI355X.

One step = rule generation + forward of one 3x3x3 submanifold convolution
64->64, fp16 storage / fp32 accumulate, on one synthetic LiDAR-like scan
(config-2 generator: 64 x 2048 x 64 range grid, ~95-120k active voxels), with
the scan (index arrays, the rows' columns, features) and the layer's weight (in the
kernel's fragment order, as a serving pipeline keeps it) already resident in HBM.
A scan of up to 1024 tiles takes ONE launch (sph_rules_conv: every workgroup makes
its tile's rules in LDS and convolves them at once), a larger one two.

The timed steps are dealt to a few HIP streams (--streams, default 3): every step redoes all
of its work into per-stream buffers, the kernels of one scan run beside those of another.
`one_stream_ms_per_step` is the same step with one scan at a time through the extension's
Python API.  The steps walk through --scans resident copies of the scan (more memory than the
last-level cache holds); the timed loop of --steps steps is repeated --repeats times and the
median counts; the untimed steps in front of a timed loop are --warmup steps and then more of
the same until --settle-ms have passed (the chip's clocks take tens of milliseconds of load to
settle, a timed loop of 20 steps lasts 0.4 ms).  `ms_per_step` is device
time (HIP events on the streams: last end - first start), `host_ms_per_step` the host's clock
around the same region between device synchronisations.

Prints ONE JSON line:  value = active voxels / second over the timed steps,
plus `rulegen_ms_per_scan`, `roofline` objects (live HIP-event timing of each kernel alone:
the step's own kernel, and the rule kernel and the convolution kernel of the two-launch path),
`mfma` (useful and executed matrix flops against the fp16 peak), an `at_120k` object (the same
step on a scan of the size BASELINE's metric names) and a `cpu_baseline` object (the CPU
restatement of the reference algorithm under oracle/, timed on this host, with the dense
conv3d of configuration 1 beside it as a sanity line).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--settle-ms", type=float, default=30.0,
                    help="untimed warm-up steps go on until this much time has passed (clocks settle); 0: only --warmup steps")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--streams", type=int, default=3, help="HIP streams the timed scans are dealt to")
    ap.add_argument("--scans", type=int, default=24,
                    help="resident copies of the scan the timed steps walk through (24 x 13 MB is more than the "
                         "256 MB last-level cache holds)")
    ap.add_argument("--repeats", type=int, default=7, help="the timed loop of `steps` steps is repeated this often; "
                                                           "the median is reported")
    ap.add_argument("--voxels", type=int, default=120000,
                    help="also measure the same step on a scan of about this many voxels (the generator's column "
                         "occupancy raised), reported as 'at_120k'; 0: skip")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--backward", action="store_true",
                    help="also time dgrad (transposed rule book + kernel) and wgrad of the same layer; "
                         "reported under 'kernels', not part of 'value'")
    ap.add_argument("--encoder", action="store_true",
                    help="also time configuration 4 (four-stage encoder, batch 4, fp16, rules regenerated every "
                         "pass) end to end; reported under 'encoder_stack', not part of 'value'")
    ap.add_argument("--callers", action="store_true",
                    help="also time the callers either side of the path (init_tensor, to_dense, xyz2RangeVoxel, "
                         "points_to_voxel_v2 + mean VFE) with HIP events; reported under 'callers'")
    ap.add_argument("--configs", action="store_true",
                    help="also time every phase (rule book, forward, dgrad, wgrad, transposed book) of the "
                         "single-layer configurations 1, 2, 3, 5a, 5b and of 8 scans of the headline grid in one "
                         "launch, one call each through the extension's Python API; reported under 'configs'")
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="budget of the CPU baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three 256 MiB device-to-device copies (a kernel of known HBM traffic, "
                         "to scale the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    ap.add_argument("--record-traffic", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: read the counter_collection.csv files of two `rocprofv3 --pmc FETCH_SIZE` / "
                         "`--pmc WRITE_SIZE` runs of `bench.py --copy-calibration --streams 1 --no-cpu-baseline` and "
                         "write profiles/hbm_traffic.json (HBM bytes per launch of the two kernels of the step at "
                         "both scan sizes, each counter scaled by what it reads for the 256 MiB copies)")
    return ap.parse_args()


def event_ms(fn, iters, torch):
    """Average duration of one fn() call: `iters` calls are enqueued back to back on
    the current stream between one pair of HIP events, so the host's launch overhead
    overlaps with the previous call's execution."""
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    # untimed calls first, for at least 30 ms: the chip's clocks take some tens of milliseconds of one kernel's
    # load to settle (the first 200 launches of a 20 us kernel read 5-7 % slower than those 25 ms later)
    t0 = time.perf_counter()
    while True:
        for _ in range(max(3, iters)):
            fn()
        torch.cuda.synchronize()
        if time.perf_counter() - t0 >= 0.03:
            break
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def cpu_baseline(d, ic, oc, budget_s, seed):
    """CPU restatement of the reference algorithm (dense-grid probe rule generation
    + per-tile gather-GEMM-scatter, fp32, OpenMP over all host cores), same scan."""
    import numpy as np
    from oracle import oracle as O
    shape, B = d["spatial_shape"], d["batch"]
    n = int(d["z_idx"].shape[0])
    rng = np.random.default_rng(seed)
    feat = rng.standard_normal((n, ic)).astype(np.float32)
    w = (rng.standard_normal((27, ic, oc)) * np.sqrt(2.0 / (27 * ic))).astype(np.float32)
    cores = len(os.sched_getaffinity(0))
    O.set_num_threads(cores)
    n_max = 256  # the reference's heuristic (80 here) overflows on clustered scans; sized not to drop pairs

    def one():
        t0 = time.perf_counter()
        _, _, rules, rule_size, dropped = O.get_rules_subm(d["z_idx"], d["z_ptr"], B, shape, shape, [3, 3, 3],
                                                           [1, 1, 1], [1, 1, 1], n_max=n_max, canonical=False)
        t1 = time.perf_counter()
        O.rule_conv(feat, w, rules, rule_size, n)
        t2 = time.perf_counter()
        return t1 - t0, t2 - t1, dropped

    for _ in range(3):  # warm-ups (the first also takes the page faults of the 1.8 GB padded rule tensor)
        one()
    times, t_start = [], time.perf_counter()
    while len(times) < 10 or (time.perf_counter() - t_start < budget_s and len(times) < 50):
        times.append(one())
    rg = sorted(t[0] for t in times)[len(times) // 2]
    fw = sorted(t[1] for t in times)[len(times) // 2]
    return {"value": n / (rg + fw), "unit": "voxels/s", "cores": cores, "kind": "port",
            "sample": "3 warm-ups, then %d scans of the same %d-voxel scan, median; rulegen %.1f ms + forward %.1f ms, "
                      "fp32, tile 2x2, tile_n_max %d, dropped pairs %d"
                      % (len(times), n, rg * 1e3, fw * 1e3, n_max, times[0][2]),
            "rulegen_ms": rg * 1e3, "forward_ms": fw * 1e3,
            "config1_sanity": config1_sanity(cores, seed)}


def config1_sanity(cores, seed):
    """Configuration 1 (64 x 512 x 32 grid, 16 -> 16 fp32) on the host: the CPU restatement (rules + forward) and,
    beside it, the dense alternative torch.nn.functional.conv3d over the whole grid.  Not the baseline."""
    import numpy as np
    import torch
    from oracle import oracle as O
    from sphconv_amd.synth import make_config
    d = make_config(1, seed=seed)
    shape, B = d["spatial_shape"], d["batch"]
    n = int(d["z_idx"].shape[0])
    rng = np.random.default_rng(seed)
    feat = rng.standard_normal((n, 16)).astype(np.float32)
    w = (rng.standard_normal((27, 16, 16)) / np.sqrt(27 * 16)).astype(np.float32)

    def sparse():
        _, _, rules, rule_size, _ = O.get_rules_subm(d["z_idx"], d["z_ptr"], B, shape, shape, [3, 3, 3], [1, 1, 1],
                                                     [1, 1, 1], canonical=False)
        return O.rule_conv(feat, w, rules, rule_size, n)

    idx = torch.tensor(d["indices"].astype(np.int64))
    dense = torch.zeros((B, 16, *shape))
    dense[idx[:, 0], :, idx[:, 1], idx[:, 2], idx[:, 3]] = torch.tensor(feat)
    wd = torch.tensor(w).reshape(3, 3, 3, 16, 16).permute(4, 3, 0, 1, 2).contiguous()
    torch.set_num_threads(cores)

    def timed(fn, reps):
        for _ in range(3):
            fn()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sorted(ts)[len(ts) // 2] * 1e3

    return {"voxels": n, "cpu_restatement_ms": timed(sparse, 10),
            "dense_conv3d_ms": timed(lambda: torch.nn.functional.conv3d(dense, wd, padding=1), 5),
            "note": "3 warm-ups, median; dense = torch conv3d over all %d cells, fp32, %d threads"
                    % (B * shape[0] * shape[1] * shape[2], cores)}


def encoder_stack_ms(torch, seed, iters):
    """Configuration 4: batch of four scans through the four-stage encoder (12 convolutions, each with
    BatchNorm(eval) + ReLU), every pass regenerates all rule books; fused tails and separate modules."""
    import numpy as np
    import sphconv_amd as sphconv
    from sphconv_amd.synth import encoder_stack, make_config
    d = make_config(4, seed=seed)
    shape, B = d["spatial_shape"], d["batch"]
    n = int(d["z_idx"].shape[0])
    dev = "cuda:0"
    rng = np.random.default_rng(seed)
    feat = torch.tensor(rng.standard_normal((n, 16)), dtype=torch.float32, device=dev).half()
    z_idx, z_ptr = torch.tensor(d["z_idx"], device=dev), torch.tensor(d["z_ptr"], device=dev)
    from sphconv_amd.rulebook import row_columns
    cols = row_columns(z_ptr, n)         # part of the tensor, as init_tensor leaves it
    net = encoder_stack(16, (16, 32, 64, 64), seed=seed).to(dev).half()
    res = {"batch": B, "voxels_in": n}

    def one():
        with torch.no_grad():
            return net(sphconv.SparseConvTensor(feat, shape, B, z_idx=z_idx, z_ptr=z_ptr, row_cols=cols))

    for fused in (True, False, True, False):             # each mode twice, the faster repeat counts
        net.fuse_eval = fused
        for _ in range(5):
            y = one()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(iters):
            y = one()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / iters * 1e3
        key = "fused_ms_per_batch" if fused else "separate_modules_ms_per_batch"
        res[key] = min(ms, res.get(key, ms))
        if fused:
            res["ms_per_scan"] = res[key] / B
            res["voxels_out"] = int(y.feature.shape[0])
    return res


def callers_ms(torch, d, seed, iters):
    """The functions either side of the convolution, each timed alone (HIP events around `iters` calls, so a
    call's own device->host read is part of its time).  `bytes` = what the call must read and write."""
    import numpy as np
    from sphconv_amd import sphconv_cuda as ext
    from sphconv_amd.data import xyz2RangeVoxel
    from sphconv_amd.synth import make_config
    from sphconv_amd.vfe import SimpleVoxel
    from sphconv_amd.voxelize import VoxelGeneratorV3
    dev = "cuda:0"
    rng = np.random.default_rng(seed)
    out = {}

    def timed(name, fn, nbytes, note):
        ms = event_ms(fn, iters, torch)
        out[name] = {"ms": ms, "bytes": nbytes, "GBps": nbytes / (ms * 1e-3) / 1e9, "workload": note}

    # COO -> compressed layout of the headline scan (rows in random order), 64 fp16 channels
    n, (S0, S1, S2), B = int(d["z_idx"].shape[0]), d["spatial_shape"], d["batch"]
    perm = rng.permutation(n)
    idx = torch.tensor(d["indices"][perm], device=dev)
    feat = torch.tensor(rng.standard_normal((n, 64)), dtype=torch.float32, device=dev).half()
    timed("init_tensor", lambda: ext.init_tensor(feat, idx, B, [S0, S1, S2]),
          n * (16 + 4 + 4 + 2 * 128) + 4 * B * S0 * S1, "%d voxels, grid %dx%dx%d, 64 fp16 channels" % (n, S0, S1, S2))
    # densify and its backward at configuration 1 (16 fp32 channels)
    c1 = make_config(1, seed=seed)
    n1, (T0, T1, T2) = int(c1["z_idx"].shape[0]), c1["spatial_shape"]
    zi1, zp1 = torch.tensor(c1["z_idx"], device=dev), torch.tensor(c1["z_ptr"], device=dev)
    f1 = torch.tensor(rng.standard_normal((n1, 16)), dtype=torch.float32, device=dev)
    dense = torch.empty((1, T0, T1, T2, 16), dtype=torch.float32, device=dev)
    timed("to_dense", lambda: ext.to_dense(f1, zi1, zp1, T2, dense), n1 * (64 + 64 + 4) + 4 * T0 * T1,
          "%d rows of 16 fp32 written into their cells of a zeroed dense %dx%dx%dx16 tensor" % (n1, T0, T1, T2))
    timed("to_dense_backward", lambda: ext.to_dense_backward(dense, zi1, zp1), n1 * (128 + 4) + 4 * T0 * T1,
          "gather of %d rows of 16 fp32 from the dense gradient" % n1)
    # one synthetic HDL-64-like sweep of the front sector: 122 880 points (x, y, z, reflectance)
    m = 64 * 1920
    theta = np.deg2rad(rng.uniform(87.5, 103.4, m))
    phi = np.deg2rad(rng.uniform(-45, 45, m))
    r = rng.uniform(6.0, 70.0, m)
    pts = np.stack([r * np.sin(theta) * np.cos(phi), r * np.sin(theta) * np.sin(phi), r * np.cos(theta),
                    rng.random(m)], 1).astype(np.float32)
    pts_d = torch.tensor(pts, device=dev)
    timed("xyz2RangeVoxel", lambda: xyz2RangeVoxel(pts_d), m * 16 + 64 * 512 * (16 + 4 + 4 + 4),
          "%d points -> range image 64x512, 512 depth bins" % m)
    gen = VoxelGeneratorV3(None, [6, -40, -3, 70.4, 40, 1], [6, -45, 87.5, 70.4, 45, 100], 2, 24000, [512, 512, 64],
                           coord_system="spherical")
    vfe = SimpleVoxel(4)

    def voxelise():
        res = gen.generate(pts_d)
        return vfe(res["voxels"], res["num_points_per_voxel"], res["coordinates"])

    timed("points_to_voxel_v2+SimpleVoxel", voxelise, m * (16 + 8 + 8) + 24000 * (2 * 16 + 8 + 12 + 4 + 16),
          "%d points -> at most 24000 voxels of 2 points on a 512x512x64 spherical grid, mean VFE" % m)
    return out


def configs_ms(torch, seed, iters):
    """Every phase of the single-layer configurations, one call each through the functions the reference's
    extension module exports (HIP events around `iters` calls; forward and dgrad include the weight pack,
    `rules` everything a rule book needs, for the strided layer its output coordinates and the one 4-byte
    device->host read).  `fwd_GBps` / `fwd_TFLOPs` price the forward's algorithmic bytes and flops."""
    from sphconv_amd import sphconv_cuda as ext
    from sphconv_amd.rulebook import RuleBook
    from sphconv_amd.synth import make_config
    dev = "cuda:0"
    out = {}

    def run(name, cfg, ic, oc, dtype, strided=False, batch=None):
        d = make_config(cfg, seed=seed, batch=batch)
        shape, B, n = d["spatial_shape"], d["batch"], int(d["z_idx"].shape[0])
        z_idx, z_ptr = torch.tensor(d["z_idx"], device=dev), torch.tensor(d["z_ptr"], device=dev)
        torch.manual_seed(seed)
        if dtype == torch.int8:
            feat = torch.randint(-20, 20, (n, ic), device=dev, dtype=torch.int8)
            w = torch.randint(-20, 20, (27, ic, oc), device=dev, dtype=torch.int8)
        else:
            feat = torch.randn((n, ic), device=dev).to(dtype)
            w = (torch.randn((27, ic, oc), device=dev) * (2.0 / (27 * ic)) ** 0.5).to(dtype)
        if strided:
            out_shape = [(s + 2 - 3) // 2 + 1 for s in shape]
            mk = lambda: RuleBook.build(z_idx, z_ptr, B, shape, out_shape, [3, 3, 3], [2, 2, 2], [1, 1, 1])
        else:
            mk = lambda: RuleBook.build_subm(z_idx, z_ptr, B, shape, [3, 3, 3])
        book = mk()
        m, P, e = book.out_rows, book.num_pairs(), feat.element_size()
        r = {"in_rows": n, "out_rows": m, "pairs": P, "channels": [ic, oc], "dtype": str(dtype).split(".")[-1],
             "rules_us": 1e3 * event_ms(mk, iters, torch)}
        if dtype == torch.int8:
            sc = torch.full((oc,), 0.01, device=dev)
            r["fwd_us"] = 1e3 * event_ms(lambda: ext.rule_conv_int8(feat, w, sc, book, None, m), iters, torch)
        else:
            r["fwd_us"] = 1e3 * event_ms(lambda: ext.rule_conv(feat, w, book, None, m), iters, torch)
            d_out = torch.randn((m, oc), device=dev).to(dtype)
            w_t = w.permute(0, 2, 1).contiguous()
            book.transposed()
            r["transposed_rules_us"] = 1e3 * event_ms(lambda: book._build(True), iters, torch)
            r["dgrad_us"] = 1e3 * event_ms(lambda: ext.rule_conv_d_feature(d_out, w_t, book, None, None, n),
                                           iters, torch)
            r["wgrad_us"] = 1e3 * event_ms(lambda: ext.rule_conv_d_weight(feat, d_out, book, None), iters, torch)
        r["fwd_GBps"] = (n * ic * e + m * oc * e + 27 * ic * oc * e + 8 * P) / r["fwd_us"] / 1e3
        r["fwd_TFLOPs"] = 2.0 * P * ic * oc / r["fwd_us"] / 1e6
        out[name] = r

    def run_refbench(name, subm, batch):
        """The reference author's benchmark shapes (test/bench_conv.py:131-133, test/Untitled.ipynb): grid
        [64, 512, 512] (512 bins on the compressed axis), 64 -> 64 fp16, real scans voxelised as the reference does."""
        import numpy as np
        import sphconv_amd as sphconv
        from sphconv_amd.synth import lidar_scan_batch
        path = os.path.join(ROOT, "tests", "golden", "kitti_000000_reduced.bin")
        if not os.path.exists(path):
            return
        shape = [64, 512, 512]
        feature, indices = lidar_scan_batch(np.fromfile(path, dtype=np.float32), batch, shape, 64, dev)
        x = sphconv.SparseConvTensor(feature, shape, batch, indices=indices)
        torch.manual_seed(seed)
        w = (torch.randn((27, 64, 64), device=dev) * (2.0 / (27 * 64)) ** 0.5).half()
        if subm:
            mk = lambda: RuleBook.build_subm(x.z_idx, x.z_ptr, batch, shape, [3, 3, 3])
        else:
            mk = lambda: RuleBook.build(x.z_idx, x.z_ptr, batch, shape, [32, 256, 256], [3, 3, 3], [2, 2, 2], [1, 1, 1])
        book = mk()
        n, m, P = int(x.feature.shape[0]), book.out_rows, book.num_pairs()
        r = {"in_rows": n, "out_rows": m, "pairs": P, "channels": [64, 64], "dtype": "float16", "batch": batch,
             "rules_us": 1e3 * event_ms(mk, iters, torch),
             "fwd_us": 1e3 * event_ms(lambda: ext.rule_conv(x.feature, w, book, None, m), iters, torch)}
        r["fwd_GBps"] = (n * 128 + m * 128 + 27 * 64 * 64 * 2 + 8 * P) / r["fwd_us"] / 1e3
        r["fwd_TFLOPs"] = 2.0 * P * 64 * 64 / r["fwd_us"] / 1e6
        out[name] = r

    run("config1_subm_16_16_f32", 1, 16, 16, torch.float32)
    run("config2_subm_32_32_f16", 2, 32, 32, torch.float16)
    run("headline_subm_64_64_f16", 2, 64, 64, torch.float16)
    run("config3_k3s2_32_64_f16_b4", 3, 32, 64, torch.float16, strided=True)
    run("config5a_subm_64_64_i8_b8", 5, 64, 64, torch.int8)
    run("config5b_subm_64_64_f16_b8", 5, 64, 64, torch.float16)
    run("headline_grid_8_scans_subm_64_64_f16", 2, 64, 64, torch.float16, batch=8)
    run_refbench("reference_bench_k3s2p1_64_64_f16_b8_grid_64x512x512", False, 8)
    run_refbench("reference_notebook_subm_64_64_f16_b3_grid_64x512x512", True, 3)
    return out


def kernel_sources_digest():
    """sha256 over the sources of the kernels whose HBM traffic is on record (what a counter run was
    taken on): the recorded traffic is only reported while these files are what it was measured on."""
    import hashlib
    h = hashlib.sha256()
    for name in ("conv.hip", "rules.hip", "fused.hip", "conv_wave.h", "rules_tile.h", "tile_consts.h", "common.h", "pack.h"):
        with open(os.path.join(ROOT, "sphconv_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def recorded_traffic(kernel_key, voxels, seed):
    """HBM bytes per launch of a kernel from profiles/hbm_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE
    scaled by a copy of known size), or None when the record is for other sources, another seed or another
    scan size."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f)
    except (OSError, ValueError):
        return None
    if rec.get("sources_sha256") != kernel_sources_digest() or rec.get("seed") != seed:
        return None
    for e in rec.get("kernels", []):
        if e.get("key") == kernel_key and e.get("voxels") == voxels:
            return e.get("hbm_bytes")
    return None


COPY_BYTES = 256 << 20      # bytes read (and written) by one --copy-calibration copy
COPY_COUNT = 3


def record_traffic(fetch_csv, write_csv, seed, voxels):
    """profiles/hbm_traffic.json from two counter runs.  A kernel's dispatches are told apart by name and grid
    size (the grid follows from the scan's tile count); the counters are KiB per dispatch, and each is scaled by
    total bytes of the calibration copies / what the counter summed to over the copy dispatches."""
    import csv
    from collections import defaultdict
    from sphconv_amd.synth import config2_with_voxels, make_config

    def load(path, counter):
        per = defaultdict(list)
        copy_sum = 0.0
        with open(path, newline="") as f:
            for r in csv.DictReader(f):
                if r["Counter_Name"] != counter:
                    continue
                name, v = r["Kernel_Name"], float(r["Counter_Value"])
                if "copyBuffer" in name and v >= 16384:    # the calibration copies, not torch's small tensor clones
                    copy_sum += v
                per[(name, int(r["Grid_Size"]))].append(v)
        if copy_sum <= 0:
            raise SystemExit("%s: no copy dispatches (run bench.py with --copy-calibration)" % path)
        factor = COPY_COUNT * COPY_BYTES / 1024.0 / copy_sum
        return per, factor

    fetch, f_fetch = load(fetch_csv, "FETCH_SIZE")
    write, f_write = load(write_csv, "WRITE_SIZE")
    sizes = [int(make_config(2, seed=seed)["z_idx"].shape[0])]
    if voxels > 0:
        sizes.append(int(config2_with_voxels(voxels, seed=seed)[0]["z_idx"].shape[0]))
    kernels = []
    for n in sizes:
        blocks = ((n + 127) // 128 + 7) // 8 * 8        # tiles, rounded up to whole rounds over the 8 XCDs
        tiles = (n + 127) // 128
        wanted = {"conv": ("conv_wave_run_kernel", lambda g: g == blocks * 192),   # wave 0 + two helper waves per tile
                  "rules": ("build_book_kernel<false>", lambda g: g == blocks * 256),
                  # one launch: workgroups of 256 threads up to 768 tiles, of 128 beyond
                  "rules_conv": ("rules_conv_kernel", lambda g: g == blocks * (256 if tiles <= 768 else 128))}
        for key, (pat, grid_ok) in wanted.items():
            def mean(per):
                vals = [v for (name, g), vs in per.items() if pat in name and grid_ok(g) for v in vs]
                if not vals:
                    raise SystemExit("no dispatch of %s for a scan of %d voxels in the counter files" % (pat, n))
                return sum(vals) / len(vals), len(vals)
            (fk, nf), (wk, nw) = mean(fetch), mean(write)
            kernels.append({"key": key, "voxels": n, "kernel": pat, "dispatches": [nf, nw],
                            "fetch_kib": round(fk, 1), "write_kib": round(wk, 1),
                            "hbm_bytes": int(round((fk * f_fetch + wk * f_write) * 1024))})
    rec = {"sources_sha256": kernel_sources_digest(), "seed": seed,
           "fetch_scale": round(f_fetch, 4), "write_scale": round(f_write, 4),
           "calibration": "%d device copies of %d MiB (--copy-calibration): bytes copied / counter sum over their "
                          "dispatches" % (COPY_COUNT, COPY_BYTES >> 20),
           "kernels": kernels}
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    with open(path, "w") as f:
        json.dump(rec, f, indent=1)
        f.write("\n")
    print(json.dumps(rec))


class Workload:
    """One scan size of the benchmark: `copies` device-resident copies of the scan (index arrays, the rows'
    columns and features in separate allocations, so that the timed steps walk through more memory than the
    256 MB last-level cache holds), and the timings of the step on it."""

    def __init__(self, torch, d, ic, oc, w, copies, seed):
        from sphconv_amd.rulebook import row_columns
        self.torch = torch
        self.d, self.ic, self.oc, self.w = d, ic, oc, w
        self.shape, self.B = d["spatial_shape"], d["batch"]
        self.n = int(d["z_idx"].shape[0])
        dev = w.device
        gen = torch.Generator(device=dev).manual_seed(seed)
        zi, zp = torch.tensor(d["z_idx"]), torch.tensor(d["z_ptr"])
        self.scans = []
        for _ in range(copies):
            feat = torch.randn((self.n, ic), device=dev, generator=gen).half()
            z_idx, z_ptr = zi.to(dev).clone(), zp.to(dev).clone()
            # the rows' columns: part of the tensor, as init_tensor and the output-coordinate kernels leave it
            self.scans.append((feat, z_idx, z_ptr, row_columns(z_ptr, self.n)))
        self.footprint = copies * (self.n * ic * 2 + self.n * 8 + zp.numel() * 4)

    def step(self, i):
        """Rule generation + forward on copy i of the scan through the extension's Python API: a rule book that
        is not built yet, and rule_conv, which makes its pairs in the launch that convolves them (the weight's
        fragment-ordered copy is kept with the weight, as for a module in eval mode)."""
        from sphconv_amd import sphconv_cuda as ext
        from sphconv_amd.rulebook import RuleBook
        feat, z_idx, z_ptr, cols = self.scans[i % len(self.scans)]
        book = RuleBook.build_subm(z_idx, z_ptr, self.B, self.shape, [3, 3, 3], row_cols=cols, lazy=True)
        book.keep = False
        return book, ext.rule_conv(feat, self.w, book, None, self.n, cache_packed=True)

    def warm(self, submit, warmup, settle_ms):
        """The untimed steps in front of a timed region: `warmup` of them, and more of the same until
        `settle_ms` have passed (the chip's clocks take some tens of milliseconds of load to settle; a timed
        region of 20 steps lasts 0.4 ms)."""
        torch = self.torch
        t0 = time.perf_counter()
        done = 0
        while True:
            for i in range(max(warmup, 20)):
                submit(done + i)
            done += max(warmup, 20)
            torch.cuda.synchronize()
            if (time.perf_counter() - t0) * 1e3 >= settle_ms:
                return

    def time_one_stream(self, steps, warmup, repeats, settle_ms=0.0):
        torch = self.torch
        with torch.no_grad():
            self.warm(self.step, warmup, settle_ms)
            times, dev_times = [], []
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            for r in range(repeats):
                t0 = time.perf_counter()
                e0.record()
                for i in range(steps):
                    self.step(r * steps + i)
                e1.record()
                torch.cuda.synchronize()
                times.append((time.perf_counter() - t0) / steps * 1e3)
                dev_times.append(e0.elapsed_time(e1) / steps)
        return sorted(dev_times)[len(dev_times) // 2], sorted(times)[len(times) // 2], dev_times

    def time_pipelined(self, steps, warmup, repeats, streams, fused=True, settle_ms=0.0):
        """The same step per scan, scans dealt to a few HIP streams so that the kernels of one scan run beside
        those of another (a 100k-voxel scan does not fill the chip); buffers are allocated once per stream slot,
        every step redoes all the work.  Device time of a repeat: from the first start to the last end over the
        streams (an event at the head of every stream's share of the steps and one at its tail, against one
        reference event); host time: the host's clock between the device synchronisations around it."""
        torch = self.torch
        from sphconv_amd.pipeline import ScanPipeline
        pipe = ScanPipeline(self.w, self.B, self.shape, max_voxels=self.n, streams=streams, fused=fused)
        if fused:
            self.step_launches = pipe.launches_for(self.n)    # what the timed step of `value` is made of

        def submit(k):
            feat, z_idx, z_ptr, cols = self.scans[k % len(self.scans)]
            return pipe.submit(feat, z_idx, z_ptr, wait_inputs=False, row_cols=cols)   # inputs are resident and complete

        self.warm(submit, warmup, settle_ms)
        pipe.synchronize()
        ns = pipe.streams
        ref = torch.cuda.Event(enable_timing=True)
        heads = [torch.cuda.Event(enable_timing=True) for _ in range(ns)]
        tails = [torch.cuda.Event(enable_timing=True) for _ in range(ns)]
        times, dev_times = [], []
        last = None
        for r in range(repeats):
            t0 = time.perf_counter()
            ref.record()
            for i in range(steps):
                slot = pipe.next_slot()
                if i < ns:
                    heads[slot].record(pipe.stream_of(slot))
                k = (r * steps + i) % len(self.scans)
                last = (submit(k), k)
                if i >= steps - ns:
                    tails[slot].record(pipe.stream_of(slot))
            torch.cuda.synchronize()      # every stream of the device (one wait, not one per stream)
            times.append((time.perf_counter() - t0) / steps * 1e3)
            used = min(ns, steps)
            slots = [(pipe.next_slot() - 1 - q) % ns for q in range(used)]
            start = min(ref.elapsed_time(heads[q]) for q in slots)
            end = max(ref.elapsed_time(tails[q]) for q in slots)
            dev_times.append((end - start) / steps)
        (out_p, _slot), k = last
        _, out = self.step(k)
        err = float((out_p.float() - out.float()).abs().max())
        assert err <= 1e-2 * max(1.0, float(out.float().abs().max())), err
        return sorted(dev_times)[len(dev_times) // 2], sorted(times)[len(times) // 2], dev_times

    def time_kernels(self, iters, backward=False, rng=None):
        """Each kernel alone: HIP events on the launch stream around `iters` back-to-back launches."""
        import ctypes as C
        from sphconv_amd import _lib as L
        from sphconv_amd import sphconv_cuda as ext
        from sphconv_amd.rulebook import RuleBook, _Buffers
        torch = self.torch
        lib = L.lib()
        feat, z_idx, z_ptr, cols = self.scans[0]
        n, ic, oc, w = self.n, self.ic, self.oc, self.w
        book = RuleBook.build_subm(z_idx, z_ptr, self.B, self.shape, [3, 3, 3], row_cols=cols)
        out = ext.rule_conv(feat, w, book, None, n)
        self.pairs = book.num_pairs()
        g = book.geom()
        bk = book.fwd.struct()
        stream = L.stream()
        zi, zp = z_idx.data_ptr(), z_ptr.data_ptr()
        res = {}
        res["rulegen_ms"] = event_ms(lambda: lib.sph_rules_build(zi, zp, n, zi, zp, n, C.byref(g), 0, C.byref(bk),
                                                                 cols.data_ptr(), stream), iters, torch)
        res["rulegen_without_columns_ms"] = event_ms(lambda: lib.sph_rules_build(zi, zp, n, zi, zp, n, C.byref(g), 0,
                                                                                 C.byref(bk), None, stream), iters, torch)
        packed = ext._packed_weight(w, False)
        out_buf = torch.empty((n, oc), dtype=torch.float16, device=w.device)
        epi = L.Epilogue(None, None, 0)
        res["conv_forward_ms"] = event_ms(lambda: lib.sph_conv_apply(L.F16, feat.data_ptr(), n, ic, packed.data_ptr(), oc,
                                                                     C.byref(bk), C.byref(epi), out_buf.data_ptr(), stream),
                                          iters, torch)
        assert torch.equal(out_buf, out)
        res["weight_pack_ms"] = event_ms(lambda: lib.sph_weight_pack(L.F16, w.data_ptr(), 27, ic, oc, ic * oc, oc, 1,
                                                                     packed.data_ptr(), stream), iters, torch)
        scratch_book = _Buffers(n, 27, w.device)
        sb = scratch_book.struct()
        one = lambda: lib.sph_rules_conv(zi, zp, n, zi, zp, n, C.byref(g), C.byref(sb), 0, cols.data_ptr(), L.F16,
                                         feat.data_ptr(), ic, packed.data_ptr(), oc, C.byref(epi), out_buf.data_ptr(), stream)
        self.one_launch = one() == 0
        if self.one_launch:
            res["rules_conv_one_launch_ms"] = event_ms(one, iters, torch)
            err = float((out_buf.float() - out.float()).abs().max())
            assert err <= 1e-2 * max(1.0, float(out.float().abs().max())), err
        if backward:
            d_out = torch.randn((n, oc), device=w.device).half()
            w_t = w.permute(0, 2, 1).contiguous()
            res["transposed_rulegen_ms"] = event_ms(lambda: book._build(True), iters, torch)
            book.transposed()
            res["dgrad_ms"] = event_ms(lambda: ext.rule_conv_d_feature(d_out, w_t, book, None, None, n), iters, torch)
            res["wgrad_ms"] = event_ms(lambda: ext.rule_conv_d_weight(feat, d_out, book, None), iters, torch)
        e, P = 2, self.pairs
        nt = book.fwd.ntiles
        self.flops = 2.0 * P * ic * oc
        self.ntiles = nt
        self.executed_groups = int(book.fwd.tile_ngrp[:nt].sum())
        self.conv_bytes = n * ic * e + n * oc * e + 27 * ic * oc * e + 8 * P
        self.rule_bytes = 4 * z_ptr.numel() + 4 * n + 4 * n + 8 * P + nt * (4 + 2 * 28)   # + the rows' columns
        # one launch: the scan and the weight in, the output rows out; the pairs never leave the chip
        self.fused_bytes = 4 * z_ptr.numel() + 4 * n + 4 * n + n * ic * e + n * oc * e + 27 * ic * oc * e
        res["rulegen_GBps"] = self.rule_bytes / (res["rulegen_ms"] * 1e-3) / 1e9
        res["conv_GBps"] = self.conv_bytes / (res["conv_forward_ms"] * 1e-3) / 1e9
        res["conv_TFLOPs"] = self.flops / (res["conv_forward_ms"] * 1e-3) / 1e12
        return res

    def _roofline(self, kernel, key, nbytes, ms, seed):
        achieved = nbytes / (ms * 1e-3) / 1e9
        return {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBS, "traffic": recorded_traffic(key, self.n, seed),
                "kernel": kernel, "algorithmic_bytes": nbytes, "kernel_ms": ms}

    def rooflines(self, kern, seed):
        """(the step's dominant kernel, the rule kernel, the convolution kernel): algorithmic bytes per launch over
        the kernel's average duration, against the HBM peak."""
        rules = self._roofline("build_book_kernel<false>", "rules", self.rule_bytes, kern["rulegen_ms"], seed)
        conv = self._roofline("conv_wave_run_kernel<f16,2,4,false>", "conv", self.conv_bytes, kern["conv_forward_ms"], seed)
        if self.one_launch and getattr(self, "step_launches", 1) == 1:
            name = "rules_conv_kernel<f16,2,4,false,%d>" % (256 if self.ntiles <= 768 else 128)
            main = self._roofline(name, "rules_conv", self.fused_bytes, kern["rules_conv_one_launch_ms"], seed)
        else:
            main = conv if kern["conv_forward_ms"] >= kern["rulegen_ms"] else rules
        return main, rules, conv

    def mfma(self, kern):
        """Matrix-unit figures of the convolution: useful flops (2 x pairs x iC x oC) over the kernel's duration
        against the fp16 MFMA peak, and what the kernel executes for them (whole groups of 16 pairs: the padding
        slots of a group are multiplied too)."""
        one = self.one_launch and getattr(self, "step_launches", 1) == 1
        ms = kern.get("rules_conv_one_launch_ms", kern["conv_forward_ms"]) if one else kern["conv_forward_ms"]
        groups = self.executed_groups
        executed = 2.0 * groups * 16 * self.ic * self.oc
        return {"useful_flops": self.flops, "executed_flops": executed, "executed_over_useful": executed / self.flops,
                "conv_kernel_TFLOPs": self.flops / (kern["conv_forward_ms"] * 1e-3) / 1e12,
                "conv_kernel_frac_of_peak": self.flops / (kern["conv_forward_ms"] * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS,
                "step_kernel_frac_of_peak": self.flops / (ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS,
                "peak_TFLOPs": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s"}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs the hot path on ONE GPU; --gpus %d is not supported "
              "(no collectives are part of this path)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    if args.record_traffic:
        record_traffic(args.record_traffic[0], args.record_traffic[1], args.seed, args.voxels)
        return
    import numpy as np
    import torch

    from sphconv_amd.synth import config2_with_voxels, make_config

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    torch.cuda.set_device(0)
    ic = oc = 64
    rng = np.random.default_rng(args.seed)
    w = torch.tensor(rng.standard_normal((27, ic, oc)) * np.sqrt(2.0 / (27 * ic)), dtype=torch.float32,
                     device=dev).half()
    d = make_config(2, seed=args.seed)

    if args.copy_calibration:
        src = torch.empty(COPY_BYTES, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(COPY_COUNT):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def measure(d):
        wl = Workload(torch, d, ic, oc, w, args.scans, args.seed)
        # the per-kernel section goes first (each kernel alone, behind 30 ms of its own launches)
        iters = max(100, min(args.steps, 200))
        kern = wl.time_kernels(iters, backward=args.backward, rng=rng)
        one_dev, one_host, one_all = wl.time_one_stream(args.steps, args.warmup, args.repeats, args.settle_ms)
        ms, host_ms, ms_all = wl.time_pipelined(args.steps, args.warmup, args.repeats, args.streams, settle_ms=args.settle_ms)
        two = wl.time_pipelined(args.steps, args.warmup, args.repeats, args.streams, fused=False, settle_ms=args.settle_ms)
        return wl, kern, {"ms": ms, "host_ms": host_ms, "one_stream_ms": one_dev, "one_stream_host_ms": one_host,
                          "two_launch_ms": two[0], "two_launch_host_ms": two[1],
                          "repeats": {"one_stream_ms": one_all, "pipelined_ms": ms_all}}

    def report(wl, kern, t):
        main_roof, rules_roof, conv_roof = wl.rooflines(kern, args.seed)
        return {"ms_per_step": t["ms"], "host_ms_per_step": t["host_ms"],
                "one_stream_ms_per_step": t["one_stream_ms"], "one_stream_host_ms_per_step": t["one_stream_host_ms"],
                "two_launch_ms_per_step": t["two_launch_ms"], "two_launch_host_ms_per_step": t["two_launch_host_ms"],
                "launches_per_step": getattr(wl, "step_launches", 1 if wl.one_launch else 2),
                "rulegen_ms_per_scan": kern["rulegen_ms"], "kernels": kern, "roofline": main_roof,
                "roofline_rules": rules_roof, "roofline_conv": conv_roof, "mfma": wl.mfma(kern), "repeats": t["repeats"]}

    wl, kern, t = measure(d)
    n, P = wl.n, wl.pairs
    rep = report(wl, kern, t)
    result = {
        "metric": "active voxels/sec, 3x3x3 subm conv 64->64 fp16 (rulegen + forward); rulegen ms/scan",
        "value": n / (rep["ms_per_step"] * 1e-3), "unit": "voxels/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "settle_ms": args.settle_ms, "ms_per_step": rep["ms_per_step"], "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": "config-2 generator (G2, seed %d): grid 64x2048x64, batch 1, %d active voxels, "
                               "%d pairs; subm 3x3x3 64->64, fp16 storage / fp32 accumulate; rules + forward in %d "
                               "launch(es) per scan; the timed steps walk through %d resident copies of the scan "
                               "(%d MB) on %d HIP streams; ms_per_step is device time (HIP events on the streams), "
                               "the median of %d repeats of `steps` steps"
                               % (args.seed, n, P, rep["launches_per_step"], args.scans, wl.footprint >> 20, args.streams,
                                  args.repeats),
                   "grid": wl.shape, "batch": wl.B, "voxels": n, "pairs": P, "channels": [ic, oc]},
        "streams": args.streams,
        "one_stream_value": n / (rep["one_stream_ms_per_step"] * 1e-3),
        "host_value": n / (rep["host_ms_per_step"] * 1e-3),
    }
    result.update({k: v for k, v in rep.items() if k != "ms_per_step"})
    if args.voxels > 0:
        # the size BASELINE's metric names: the same generator with its column occupancy raised
        d2, p2 = config2_with_voxels(args.voxels, seed=args.seed)
        wl2, kern2, t2 = measure(d2)
        rep2 = report(wl2, kern2, t2)
        result["at_120k"] = {
            "workload": "config-2 generator with column occupancy %.3f: %d active voxels, %d pairs" % (p2, wl2.n, wl2.pairs),
            "voxels": wl2.n, "pairs": wl2.pairs, "value": wl2.n / (rep2["ms_per_step"] * 1e-3), "unit": "voxels/s"}
        result["at_120k"].update(rep2)
    if args.callers:
        result["callers"] = callers_ms(torch, d, args.seed, 50)
    if args.configs:
        result["configs"] = configs_ms(torch, args.seed, 30)
    if args.encoder:
        result["encoder_stack"] = encoder_stack_ms(torch, args.seed, 20)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(d, ic, oc, args.cpu_seconds, args.seed)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
