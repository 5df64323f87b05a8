"""Benchmark of the IVF-PQ search path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config N]

One step = one `cuvsIvfPqSearch` call over the whole query batch with the queries already in HBM.
Workload (BASELINE.json configs[2], the configuration the metric is quoted on): 10M x 128 uint8
SIFT-like rows, n_lists = 16384, pq_dim = 64, pq_bits = 8, 10,000 queries, k = 10, n_probes = 64,
fp16 lookup table with fp32 internal distances.  Prints ONE JSON line with the QPS and recall@10 of the
library's default path, the roofline of the code-scan kernel and a CPU baseline (the oracle,
multithreaded, on a bounded query sample).

The roofline is the one the metric defines: algorithmic bytes of the code stream = sum over all
(query, probed list) pairs of round_up(list size, 32) * bytes per encoded row, over the duration of
the kernel that streams them.  The default path does not stream those bytes for L2 metrics (it
drops most pairs after their leading codes), so the same batch is also run with the early stop
switched off on the handle (cuvsAmdIvfPqSetSearchTuning): one launch of the scan kernel over every
probed list in full, timed with HIP events on the library's stream.  `roofline` is that launch;
`default_path` holds the launches of the path that `value` was measured on.

`--config N` (0..4) runs another of BASELINE.json's configurations at its real shape instead (same
JSON line; the CPU baseline only with `--with-cpu`, since copying a large index to the host takes
longer than the benchmark).  Single flags (`--probes 128`, `--k 100`, `--lut fp8`, `--queries 100`
...) override the configuration's values.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E

# BASELINE.json's configurations; `dataset` names the generator below
CONFIGS = {
    0: dict(rows=10_000, lists=64, queries=100, probes=8, dim=128, pq_dim=32, pq_bits=8, k=10, lut="f32",
            internal="f32", metric="sqeuclidean", kind="subspace", dataset="mixture64_f32"),
    1: dict(rows=1_000_000, lists=1024, queries=10_000, probes=32, dim=96, pq_dim=48, pq_bits=8, k=10,
            lut="f16", internal="f32", metric="sqeuclidean", kind="subspace", dataset="unit_mixture_f32"),
    2: dict(rows=10_000_000, lists=16384, queries=10_000, probes=64, dim=128, pq_dim=64, pq_bits=8, k=10,
            lut="f16", internal="f32", metric="sqeuclidean", kind="subspace", dataset="sift_u8"),
    3: dict(rows=10_000_000, lists=16384, queries=10_000, probes=64, dim=768, pq_dim=384, pq_bits=4, k=10,
            lut="fp8", internal="f16", metric="inner_product", kind="subspace", dataset="decay_mixture_f32"),
    4: dict(rows=100_000_000, lists=50_000, queries=10_000, probes=200, dim=96, pq_dim=48, pq_bits=8, k=10,
            lut="f16", internal="f32", metric="sqeuclidean", kind="cluster", dataset="mixture_f16"),
}


def make_rows(name, n, dim, device):
    """Synthetic rows of BASELINE.json's configurations (seeded)."""
    import torch

    import datasets as testing
    if name == "sift_u8":
        return testing.sift_like_u8(n, dim, 4096, seed=1234, device=device)
    if name == "mixture64_f32":
        return testing.gaussian_mixture(n, dim, 64, 0.3, seed=1234, device=device)
    if name == "unit_mixture_f32":
        return testing.gaussian_mixture(n, dim, 1000, 0.2, seed=1234, device=device, normalize_centers=True,
                                        normalize_rows=True)
    if name == "decay_mixture_f32":
        return testing.gaussian_mixture(n, dim, 8192, 0.3, seed=1234, device=device, dim_decay=0.9,
                                        normalize_rows=True)
    if name == "mixture_f16":
        return testing.gaussian_mixture(n, dim, 50_000, 0.25, seed=1234, device=device, dtype=torch.float16)
    raise ValueError(name)


def log(msg):
    print(f"[bench {time.strftime('%H:%M:%S')}] {msg}", file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--rows", type=int, default=10_000_000)
    ap.add_argument("--lists", type=int, default=16384)
    ap.add_argument("--queries", type=int, default=10_000)
    ap.add_argument("--probes", type=int, default=64)
    ap.add_argument("--dim", type=int, default=128)
    ap.add_argument("--pq-dim", type=int, default=64)
    ap.add_argument("--pq-bits", type=int, default=8)
    ap.add_argument("--k", type=int, default=10)
    ap.add_argument("--lut", default="f16", choices=["f32", "f16", "fp8"])
    ap.add_argument("--internal", default="f32", choices=["f32", "f16"])
    ap.add_argument("--build", choices=("native", "torch"), default="native",
                    help="train the index with the library (cuvsIvfPqBuild) or with the torch helper")
    ap.add_argument("--refine-ratio", type=int, default=1,
                    help="search refine_ratio * k candidates and re-rank them exactly (1 = off)")
    ap.add_argument("--early-stop", choices=("auto", "off", "on"), default="auto",
                    help="fix the library's choice of the L2 early stop for the whole run (profiling runs)")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-sweep", action="store_true",
                    help="skip the `sweep` entries (other search parameters and workloads, 5 steps each) that the "
                         "default run appends to its JSON line")
    ap.add_argument("--with-cpu", action="store_true", help="time the CPU oracle also with --config")
    ap.add_argument("--config", type=int, default=2, choices=sorted(CONFIGS))
    ap.add_argument("--metric", default="sqeuclidean", choices=["sqeuclidean", "euclidean", "inner_product", "cosine"])
    ap.add_argument("--kind", default="subspace", choices=["subspace", "cluster"])
    ap.add_argument("--dataset", default="sift_u8")
    first, _ = ap.parse_known_args()
    ap.set_defaults(**CONFIGS[first.config])
    args = ap.parse_args()
    if args.config != 2 and not args.with_cpu:
        args.no_cpu = True
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import numpy as np
    import torch

    import datasets as testing

    from cuvs_amd import ivf_pq, refine
    from cuvs_amd.resources import Resources

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda"
    dim, pq_dim, pq_bits = args.dim, args.pq_dim, args.pq_bits
    n, nq, n_lists, P, k = args.rows, args.queries, args.lists, args.probes, args.k
    lut_np = {"f32": np.float32, "f16": np.float16, "fp8": np.uint8}[args.lut]
    int_np = {"f32": np.float32, "f16": np.float16}[args.internal]

    t0 = time.time()
    allrows = make_rows(args.dataset, n + nq, dim, dev)
    data, queries = allrows[:n], allrows[n:].contiguous()
    torch.cuda.synchronize()
    log(f"data {tuple(data.shape)} {str(data.dtype).replace('torch.', '')} ({args.dataset}) generated in "
        f"{time.time() - t0:.1f}s")

    res = Resources()
    res.use_torch_current_stream()
    res.set_search_tuning(early_stop=args.early_stop)
    n_train = min(n, max(n_lists * 32, 200_000))
    if args.build == "native":
        # the library's own training (cuvsIvfPqBuild) on a subsample of n_train rows, then every row
        # encoded and added (add_data_on_build)
        t0 = time.time()
        params = ivf_pq.IndexParams(n_lists=n_lists, metric=args.metric, pq_bits=pq_bits, pq_dim=pq_dim,
                                    codebook_kind=args.kind,
                                    kmeans_trainset_fraction=min(1.0, n_train / n))
        index = ivf_pq.build(params, data, resources=res)
        res.sync()
        model = {"centers": index.centers_padded, "centers_rot": index.centers_rot,
                 "rotation_matrix": index.rotation_matrix, "pq_centers": index.pq_centers}
        log(f"index trained on ~{n_train} rows and populated ({len(index)} rows) in {time.time() - t0:.1f}s")
    else:
        assert (args.metric, args.kind, args.dataset) == ("sqeuclidean", "subspace", "sift_u8"), \
            "--build torch covers the default workload only"
        t0 = time.time()
        g = torch.Generator(device="cpu")
        g.manual_seed(137)
        sel = torch.randperm(n, generator=g)[:n_train].to(dev)
        model = testing.train_model(data[sel], n_lists, pq_dim, pq_bits, kmeans_iters=6, pq_iters=8,
                                    seed=137, half_assign=True)
        torch.cuda.synchronize()
        log(f"model trained on {n_train} rows in {time.time() - t0:.1f}s")

        t0 = time.time()
        labels = testing.assign_nearest(data, model["centers"][:, :dim], half=True).to(torch.int32)
        torch.cuda.synchronize()
        log(f"lists assigned in {time.time() - t0:.1f}s")

        t0 = time.time()
        params = ivf_pq.IndexParams(n_lists=n_lists, pq_bits=pq_bits, pq_dim=pq_dim)
        index = ivf_pq.build_precomputed(params, dim, model["pq_centers"], model["centers"],
                                         model["centers_rot"], model["rotation_matrix"], resources=res)
        ivf_pq.extend(index, data, None, resources=res, labels=labels)
        res.sync()
        log(f"index populated ({len(index)} rows) in {time.time() - t0:.1f}s")

    t0 = time.time()
    truth = testing.exact_knn(data, queries, k, metric=args.metric).cpu().numpy()  # fp32: exact for 8-bit data
    log(f"exact ground truth in {time.time() - t0:.1f}s")

    sp = ivf_pq.SearchParams(n_probes=P, lut_dtype=lut_np, internal_distance_dtype=int_np,
                             max_internal_batch_size=max(nq, 1))
    k_search = k * max(args.refine_ratio, 1)
    neighbors = torch.empty((nq, k_search), dtype=torch.int64, device=dev)
    distances = torch.empty((nq, k_search), dtype=torch.float32, device=dev)
    refined_ids = torch.empty((nq, k), dtype=torch.int64, device=dev)
    refined_d = torch.empty((nq, k), dtype=torch.float32, device=dev)

    def step():
        ivf_pq.search(sp, index, queries, k_search, neighbors=neighbors, distances=distances,
                      resources=res)
        if args.refine_ratio > 1:
            refine(data, queries, neighbors, k, metric=args.metric, indices=refined_ids,
                   distances=refined_d, resources=res)

    # the first search on a new index runs the early-stop screen where the shapes allow it and is
    # observed; where the screen kept most pairs, the searches after it scan plainly
    res.enable_profiling(True)
    step()
    first_call_screened = ivf_pq.get_search_profile(res)["n_screened_pairs"] > 0
    res.enable_profiling(False)
    res.sync()
    for _ in range(args.warmup):
        step()
    res.sync()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    res.sync()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    qps = nq * args.steps / elapsed
    gpu_ids = (refined_ids if args.refine_ratio > 1 else neighbors).cpu().numpy()
    gpu_recall = testing.recall(gpu_ids, truth)
    log(f"{ms_per_step:.2f} ms per batch of {nq}: {qps:,.0f} QPS, recall@{k} {gpu_recall:.4f}")

    # per-kernel times of the scan stage: HIP events on the library's stream, same steps again
    def profiled(steps):
        res.enable_profiling(True)
        prof = []
        for _ in range(steps):
            step()
            prof.append(ivf_pq.get_search_profile(res))
        res.enable_profiling(False)
        return prof

    def timed(steps, warmup):
        for _ in range(warmup):
            step()
        res.sync()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        res.sync()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    prof = profiled(args.steps)
    stage = prof[-1]
    launches = max(stage["n_scan_launches"], 1)
    mean = lambda pr, f: float(np.mean([p[f] for p in pr]))
    scan_bytes = float(stage["scan_bytes"])  # all probed lists in full, summed on the device from the probe lists
    early_stop = stage["n_screened_pairs"] > 0
    # the kernel that scans pairs in full, as the library reports it
    KERNELS = {0: "scan_kernel", 1: "scan_stream_kernel", 2: "scan_fast_kernel", 3: "scan_direct_kernel",
               4: "scan_nibble_kernel", 5: "scan_nibble_pack_kernel", 6: "scan_slab_kernel"}
    full_name = KERNELS[stage["scan_kernel"]]
    if first_call_screened and not early_stop:
        log("the screen kept most pairs on the first search: it is off for the searches after it")
    default_path = {"early_stop": bool(early_stop), "screen_switched_itself_off": bool(first_call_screened and not early_stop),
                    "ms_per_step": ms_per_step, "qps": qps,
                    "scan_stage_ms": mean(prof, "scan_ms"),
                    "stage_ms": {s_: mean(prof, s_) for s_ in ("coarse_ms", "rotate_ms", "scan_ms", "merge_ms")}}
    if early_stop:
        # three launches: the leading probes' lists in full, the screen of every other pair on its
        # 8 leading codes (8 bytes a row), the surviving pairs in full
        screen_name = "scan_screen_kernel" if args.kind == "cluster" else "scan_screen_direct_kernel"
        parts = {"lead_scan": (full_name, mean(prof, "lead_scan_ms"), float(stage["lead_bytes"])),
                 "screen": (screen_name, mean(prof, "screen_ms"), float(stage["screen_bytes"])),
                 "survivor_scan": (full_name, mean(prof, "survivor_scan_ms"), float(stage["survivor_bytes"]))}
        default_path["launches"] = {
            name: {"kernel": kn, "ms": ms, "bytes_read_by_the_algorithm": b,
                   "rate_on_those_bytes_GBs": b / (ms * 1e-3) / 1e9 if ms > 0 else None}
            for name, (kn, ms, b) in parts.items()}
        default_path["launches"]["screen"]["note"] = (
            "8 bytes per padded row of every screened pair: a unit of this library's own, served "
            "largely from L2 (pairs run in list order), not the metric's code stream")
        default_path["pairs_screened"] = int(stage["n_screened_pairs"])
        default_path["pairs_surviving"] = int(stage["n_surviving_pairs"])
        default_path["pairs_dropped_on_their_length"] = int(stage["n_far_pairs"])
        if stage["n_far_pairs"]:
            # the bytes are those of every screened pair; most were never read
            default_path["launches"]["screen"]["rate_on_those_bytes_GBs"] = None
            default_path["launches"]["screen"]["kernel"] = (
                "far_query_terms_kernel, far_count_kernel, far_move_kernel; then " + screen_name +
                " over the pairs they leave, unless the index has found that it keeps most of them")
        default_path["launches"]["screen"]["note"] += (
            "; pairs whose |query - centre| minus the list's radius lies past the query's bound are "
            "dropped without reading a row, and their rows are counted here all the same")
        log("default path, scan stage: " + ", ".join(f"{n_} {ms:.3f} ms / {b / 1e9:.2f} GB"
                                                     for n_, (_, ms, b) in parts.items())
            + f"; {stage['n_surviving_pairs']} of {stage['n_screened_pairs']} screened pairs kept "
            f"({stage['n_far_pairs']} dropped without reading a row); "
            f"all probed lists in full are {scan_bytes / 1e9:.2f} GB")

    # The code stream in full: the same batch with the early stop switched off on the handle.  One
    # launch of the scan kernel per internal batch reads every probed list.
    if early_stop:
        res.set_search_tuning(early_stop="off")
        full_ms_per_step = timed(args.steps, args.warmup)
        full_prof = profiled(args.steps)
        full_ids = neighbors.cpu().numpy().copy()
        res.set_search_tuning(early_stop=args.early_stop)
        assert full_prof[-1]["n_screened_pairs"] == 0
        same_ids = bool((full_ids == gpu_ids).all()) if args.refine_ratio <= 1 else None
    else:
        full_ms_per_step, full_prof, same_ids = ms_per_step, prof, None
    full_name = KERNELS[full_prof[-1]["scan_kernel"]]
    full_launches = max(full_prof[-1]["n_scan_launches"], 1)
    kernel_ms = mean(full_prof, "scan_ms") / full_launches
    kernel_bytes = float(full_prof[-1]["scan_bytes"]) / full_launches
    achieved = kernel_bytes / (kernel_ms * 1e-3) / 1e9
    default_workload = (args.config == 2 and n == 10_000_000 and dim == 128 and n_lists == 16384 and pq_dim == 64 and
                        pq_bits == 8 and nq == 10_000 and k == 10 and P == 64 and args.lut == "f16" and
                        args.internal == "f32" and args.metric == "sqeuclidean" and args.kind == "subspace" and
                        full_name == "scan_stream_kernel")
    traffic = 1.67e9 if default_workload else None  # 1.46 GB fetched + 0.21 GB written per launch
    traffic_source = ("profiles/scan_stream_kernel_configs2_configs1_counters.md" if default_workload else None)
    log(f"code stream in full: {full_name} {kernel_ms:.3f} ms per launch, {kernel_bytes / 1e9:.2f} GB algorithmic "
        f"-> {achieved:.0f} GB/s ({achieved / HBM_PEAK_GBS:.1%} of HBM peak); {full_ms_per_step:.2f} ms per batch = "
        f"{nq / full_ms_per_step * 1e3:,.0f} QPS" + (f"; ids identical to the default path: {same_ids}" if same_ids is not None else ""))

    # the reference's default max_internal_batch_size (4096): what a drop-in caller gets
    sp_saved = sp
    default_batching = None
    if nq > 4096:
        sp = ivf_pq.SearchParams(n_probes=P, lut_dtype=lut_np, internal_distance_dtype=int_np)
        ms_4096 = timed(args.steps, args.warmup)
        default_batching = {"max_internal_batch_size": 4096, "ms_per_step": ms_4096, "qps": nq / ms_4096 * 1e3}
        log(f"max_internal_batch_size = 4096 (the reference's default): {ms_4096:.2f} ms per batch = "
            f"{nq / ms_4096 * 1e3:,.0f} QPS")
        sp = sp_saved

    # A plain copy of known size (1 GiB read + 1 GiB written), outside every timed region: it gives
    # hardware-counter runs of this same command the reading of FETCH_SIZE / WRITE_SIZE per byte.
    calib = torch.zeros(2 ** 28, dtype=torch.int32, device=dev)
    calib_out = torch.empty_like(calib)
    torch.add(calib, 1, out=calib_out)
    torch.cuda.synchronize()
    del calib, calib_out

    out = {
        "metric": ("QPS@recall@10 (10M x 128 IVF-PQ, batch 10k); code-scan HBM GB/s vs peak" if args.config == 2
                   else f"QPS@recall@{k} ({n} x {dim} IVF-PQ, batch {nq}); code-scan HBM GB/s vs peak"),
        "value": qps, "unit": "queries/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32" if args.internal == "f32" else "f16",
        "data": "synthetic",
        "config": {"workload": f"configs[{args.config}]: {n} x {dim} {str(data.dtype).replace('torch.', '')} "
                               f"({args.dataset}), n_lists={n_lists}, pq_dim={pq_dim}, pq_bits={pq_bits}, "
                               f"{args.kind} codebooks, {nq} queries, k={k}, n_probes={P}, lut={args.lut}, "
                               f"internal={args.internal}, {args.metric}",
                   "n_rows": n, "dim": dim, "n_lists": n_lists, "pq_dim": pq_dim,
                   "pq_bits": pq_bits, "n_queries": nq, "k": k, "n_probes": P,
                   "lut_dtype": args.lut, "internal_distance_dtype": args.internal,
                   "refine_ratio": args.refine_ratio,
                   "recall_at_k": gpu_recall},
        # the code-scan kernel streaming every probed list in full: algorithmic bytes as the metric
        # defines them over the HIP-event time of that one launch; HBM traffic comes from hardware
        # counters, which this script does not read: for the default workload it is the figure of
        # the counter runs kept under profiles/ (FETCH_SIZE x 2.0 + WRITE_SIZE x 1.0, the factors a
        # 1 GiB copy reads in the same runs), for any other workload null
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "traffic_source": traffic_source,
                     "kernel": full_name, "kernel_ms": kernel_ms,
                     "algorithmic_bytes_per_launch": kernel_bytes,
                     "path": ("early stop switched off on the handle: every probed list streamed in full"
                              if early_stop else "the default path streams every probed list in full"),
                     "ms_per_step_on_this_path": full_ms_per_step,
                     "qps_on_this_path": nq / full_ms_per_step * 1e3,
                     "ids_identical_to_default_path": same_ids},
        "default_path": default_path,
    }
    if default_batching is not None:
        out["default_batching"] = default_batching

    if not args.no_cpu and args.refine_ratio <= 1:
        out["cpu_baseline"] = cpu_baseline(args, index, model, queries, truth, gpu_ids, dim, pq_dim,
                                           pq_bits, P, k, log)
        out["config"]["oracle_recall_on_sample"] = out["cpu_baseline"].pop("oracle_recall")
        out["config"]["gpu_recall_on_sample"] = out["cpu_baseline"].pop("gpu_recall")
    default_run = args.config == 2 and (n, dim, pq_dim, pq_bits, nq, n_lists, P, k) == (
        10_000_000, 128, 64, 8, 10_000, 16384, 64, 10) and args.refine_ratio <= 1
    if default_run and not args.no_sweep:
        out["sweep"] = sweep(args, res, index, data, queries, log)
    print(json.dumps(out), flush=True)


def measure_variant(res, index, queries, truth, k, P, lut, internal, steps, warmup, workload):
    """One sweep entry: the default path's time per batch and recall, and the code-scan kernel of
    the same batch with the early stop off (every probed list streamed in full) against the HBM
    peak, as `roofline` does for the headline."""
    import numpy as np
    import torch

    import datasets as testing
    from cuvs_amd import ivf_pq

    lut_np = {"f32": np.float32, "f16": np.float16, "fp8": np.uint8}[lut]
    int_np = {"f32": np.float32, "f16": np.float16}[internal]
    nq = queries.shape[0]
    sp = ivf_pq.SearchParams(n_probes=P, lut_dtype=lut_np, internal_distance_dtype=int_np,
                             max_internal_batch_size=max(nq, 1))
    neighbors = torch.empty((nq, k), dtype=torch.int64, device="cuda")
    distances = torch.empty((nq, k), dtype=torch.float32, device="cuda")

    def step():
        ivf_pq.search(sp, index, queries, k, neighbors=neighbors, distances=distances, resources=res)

    def timed():
        for _ in range(warmup):
            step()
        res.sync()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        res.sync()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    res.set_search_tuning(early_stop="auto")
    step()  # the first search with new parameters is the one the screen's feedback observes
    res.sync()
    ms = timed()
    ids = neighbors.cpu().numpy().copy()
    res.enable_profiling(True)
    step()
    default_prof = ivf_pq.get_search_profile(res)
    res.set_search_tuning(early_stop="off")
    prof = []
    for _ in range(steps):
        step()
        prof.append(ivf_pq.get_search_profile(res))
    res.enable_profiling(False)
    res.set_search_tuning(early_stop="auto")
    same = bool((neighbors.cpu().numpy() == ids).all())
    launches = max(prof[-1]["n_scan_launches"], 1)
    kernel_ms = float(np.mean([p_["scan_ms"] for p_ in prof])) / launches
    kernel_bytes = float(prof[-1]["scan_bytes"]) / launches
    achieved = kernel_bytes / (kernel_ms * 1e-3) / 1e9
    kernels = {0: "scan_kernel", 1: "scan_stream_kernel", 2: "scan_fast_kernel", 3: "scan_direct_kernel",
               4: "scan_nibble_kernel", 5: "scan_nibble_pack_kernel", 6: "scan_slab_kernel"}
    return {"workload": workload, "ms_per_step": ms, "qps": nq / ms * 1e3,
            "recall": testing.recall(ids, truth), "early_stop_on_default_path": default_prof["n_screened_pairs"] > 0,
            "kernel": kernels[prof[-1]["scan_kernel"]], "kernel_ms": kernel_ms,
            "algorithmic_bytes": kernel_bytes, "achieved_GBs": achieved, "frac": achieved / HBM_PEAK_GBS,
            "ids_identical_to_default_path": same}


def sweep(args, res, index, data, queries, log):
    """Other search parameters on the headline index, and two other workloads, 5 steps each: the
    figures that do not depend on how well the headline rows cluster."""
    import torch

    import datasets as testing
    from cuvs_amd import ivf_pq

    steps, warmup = 5, 2
    entries = []

    def add(res_, index_, queries_, truth_, k, P, lut, internal, workload):
        e = measure_variant(res_, index_, queries_, truth_, k, P, lut, internal, steps, warmup, workload)
        log(f"sweep: {workload}: {e['ms_per_step']:.2f} ms per batch, recall {e['recall']:.4f}; {e['kernel']} "
            f"{e['kernel_ms']:.3f} ms for {e['algorithmic_bytes'] / 1e9:.2f} GB = {e['frac']:.3f} of HBM peak")
        entries.append(e)

    truth10 = testing.exact_knn(data, queries, 10, metric=args.metric).cpu().numpy()
    truth100 = testing.exact_knn(data, queries, 100, metric=args.metric).cpu().numpy()
    head = "configs[2] (10M x 128 u8, 16384 lists, pq_dim 64)"
    add(res, index, queries, truth10, 10, 64, "fp8", "f32", head + ", k=10, n_probes=64, fp8 table")
    add(res, index, queries, truth100, 100, 64, "f16", "f32", head + ", k=100, n_probes=64, fp16 table")
    add(res, index, queries, truth10, 10, 128, "f16", "f32", head + ", k=10, n_probes=128, fp16 table")
    add(res, index, queries, truth10, 10, 64, "f32", "f32",
        head + ", k=10, n_probes=64, fp32 table (the reference's default lut_dtype)")

    def other(dataset, rows, dim, lists, pq_dim, P, variants):
        """variants: (lut, workload) pairs measured on one index"""
        nq = queries.shape[0]
        allrows = make_rows(dataset, rows + nq, dim, "cuda")
        x, q = allrows[:rows], allrows[rows:].contiguous()
        params = ivf_pq.IndexParams(n_lists=lists, metric="sqeuclidean", pq_bits=8, pq_dim=pq_dim,
                                    kmeans_trainset_fraction=min(1.0, max(lists * 32, 200_000) / rows))
        ix = ivf_pq.build(params, x, resources=res)
        res.sync()
        truth = testing.exact_knn(x, q, 10, metric="sqeuclidean").cpu().numpy()
        for lut, workload in variants:
            add(res, ix, q, truth, 10, P, lut, "f32", workload)
        del ix, x, q, allrows
        torch.cuda.empty_cache()

    c1 = "configs[1] (1M x 96 f32 unit vectors, 1024 lists, pq_dim 48), k=10, n_probes=32, "
    other("unit_mixture_f32", 1_000_000, 96, 1024, 48, 32, [("f16", c1 + "fp16 table"), ("fp8", c1 + "fp8 table")])
    other("sift_u8", 2_000_000, 256, 2048, 128, 32,
          [("f16", "2M x 256 u8 (sift_u8), 2048 lists, pq_dim 128 (the reference's default pq_dim for 256 dimensions), "
            "k=10, n_probes=32, fp16 table")])
    other("sift_u8", 1_000_000, 768, 1024, 384, 32,
          [("f16", "1M x 768 u8 (sift_u8), 1024 lists, pq_dim 384 (the reference's default pq_dim for 768 dimensions), "
            "k=10, n_probes=32, fp16 table")])
    return entries


def cpu_baseline(args, index, model, queries, truth, gpu_ids, dim, pq_dim, pq_bits, P, k, log):
    """The CPU oracle (a scalar restatement of the reference algorithm, multithreaded over
    queries) timed on a bounded sample of the same queries against the same index contents."""
    import numpy as np

    import gpu_helpers as G
    import datasets as testing
    from oracle import oracle

    t0 = time.time()
    host_model = {kk: v.cpu().numpy() for kk, v in model.items()}
    ix = G.read_back_bulk(oracle, index, host_model, dim, pq_dim, pq_bits, args.metric, args.kind)
    log(f"index copied to the host for the CPU baseline in {time.time() - t0:.1f}s")
    lut = {"f32": 0, "f16": 2, "fp8": 8}[args.lut]
    internal = {"f32": 0, "f16": 2}[args.internal]
    threads = oracle.default_threads()
    q_host = queries.cpu().numpy()
    pilot = min(2 * threads, q_host.shape[0])
    t0 = time.perf_counter()
    oracle.search(ix, q_host[:pilot], k, P, lut_dtype=lut, internal_distance_dtype=internal,
                  n_threads=threads)
    per_query = (time.perf_counter() - t0) / pilot
    n_sample = int(min(q_host.shape[0], max(pilot, args.cpu_seconds / max(per_query, 1e-9))))
    t0 = time.perf_counter()
    nb, _ = oracle.search(ix, q_host[:n_sample], k, P, lut_dtype=lut,
                          internal_distance_dtype=internal, n_threads=threads)
    dt = time.perf_counter() - t0
    o_rec = testing.recall(nb, truth[:n_sample])
    g_rec = testing.recall(gpu_ids[:n_sample], truth[:n_sample])
    same = float((nb == gpu_ids[:n_sample]).mean())
    log(f"CPU oracle: {n_sample} queries in {dt:.1f}s on {threads} threads = {n_sample / dt:,.0f} QPS; "
        f"recall {o_rec:.4f} (GPU on the same queries {g_rec:.4f}); identical ids {same:.4%}")
    return {"value": n_sample / dt, "unit": "queries/s", "cores": threads, "kind": "port",
            "sample": f"first {n_sample} of the {q_host.shape[0]} queries, same index and parameters",
            "oracle_recall": o_rec, "gpu_recall": g_rec, "ids_identical_frac": same}


if __name__ == "__main__":
    main()
