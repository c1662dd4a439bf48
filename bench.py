#!/usr/bin/env python3
"""Benchmark of the collection path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

Workload (N=1): Pythia-160m-shaped GPT-NeoX, random-init bf16; 2048 documents with lengths
lognormal(6, 1) clipped to [16, 2048], bin-packed into 4096-token batches, uniform-random ids;
projection_dim 16 Gaussian projections on all 48 Linear modules; Adafactor normalizer with second
moments |N(0,1)| * 1e-4; per-sequence gradients written to an fp16 store.

A step is one batch through the whole path: padding and upload of the token ids, forward, loss, backward
(hooks queue the modules), one fused collection launch into the device-resident fp16 store.  The timed
region is `CollectorComputer.run_with_collector_hooks` over the K timed batches as a whole -- the reference's
own definition (benchmarks/benchmark_bergson.py:355-358: tokens / seconds of the build loop) -- so it also
holds the store flush to its memory-mapped file, the loss column and the processor files written by
`teardown()`.  value = documents' tokens / wall seconds.  `prestaged` is the same K batches once more with the
padded batches already in HBM and only the store flush behind the loop (what earlier records called value).

One JSON line is printed.  It also carries
  roofline      the fused collection kernel: algorithmic bytes (a and g read once) per launch over its
                duration measured with events on the launch stream, against 8 TB/s;
  cpu_baseline  the CPU oracle (the reference's op sequence on PyTorch CPU) on a bounded sample;
  gpu_torch_baseline  the same op sequence as cpu_baseline issued as stock PyTorch-ROCm ops on this GPU (module
                hooks, elementwise scale, skinny GEMMs, bmm, clamp, cat): what the fused launch replaces;
  store_scan    the second half of the metric: 10^6 fp16 rows of 12288 scanned against 1024 queries
                with unit-norm cosine, top-100 per query and the per-row max; its own cpu_baseline is the
                reference's search on a slice of the store;
  per_token     configs[1]'s modules with one row per token (attribute_tokens), kernel only;
  wide_projection  configs[1]'s modules with per-sequence rows at p = 32 and p = 64, kernel only;
  llama8b_layers  configs[4]'s module shapes through a 4-layer Llama-3-8B-shaped model;
  adam_per_token  configs[3]'s hot kernel, and `end_to_end`: the product loop on a Pythia-410m-shaped model over a
                slice of that configuration, into the real 98 304-wide per-token store;
  config1       configs[0], the one configuration the reference's CPU path runs, in full on both sides: the product
                loop on the GPU and the oracle loop on the host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import tempfile
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0
# HBM bytes moved per algorithmic byte by collect_kernel on this workload, from the FETCH_SIZE and
# WRITE_SIZE hardware counters (profiles/collect_and_scan_kernels_pmc_hbm_traffic.txt)
COLLECT_TRAFFIC_RATIO = 1.036
# the same for the store scan: 1024 queries (rows once; the 25 MB of queries once per round of 24 576 rows and XCD),
# at most 32 queries; and for per-token collection and the Llama-3-8B-shaped layers
SCAN_TRAFFIC_RATIO_Q1024 = 1.345
SCAN_TRAFFIC_RATIO_FEW = 1.0016
PER_TOKEN_TRAFFIC_RATIO = 1.068
WIDE_TRAFFIC_RATIO = {32: 1.078, 64: 1.151}
WIDE_TOK_TRAFFIC_RATIO = 1.113
LLAMA_TRAFFIC_RATIO = 0.994
# bytes the four fused Adam launches of one layer fetch through the L2s and write, from the same counters
# (profiles/adam_fused_pythia410m_layer_p32.txt): 5.19 GB + 0.07 GB, against 0.94 GB read once each
ADAM_TRAFFIC_BYTES_PER_LAYER = 5.26e9
MFMA_F16_PEAK_TFLOPS = 2500.0


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=260,
                    help="timed batches (default: 260 of the workload's 323, so that the store flush at the end and the "
                         "pipeline's first and last half-steps weigh about what they weigh in a whole run)")
    ap.add_argument("--warmup", type=int, default=60,
                    help="untimed batches first (default 60: in a fresh process the first ~50 batches of new shapes run "
                         "at 12 ms instead of 8.8: the libraries under the model load kernels and pick GEMM variants "
                         "on first use)")
    ap.add_argument("--docs", type=int, default=2048)
    ap.add_argument("--token-batch-size", type=int, default=4096)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-scan", action="store_true",
                    help="skip every leg but the headline one (store scan, per-token, Llama shapes, Adam)")
    ap.add_argument("--scan-only", action="store_true",
                    help="run the store-scan leg alone and print its entry (for counter runs on the scan kernels)")
    ap.add_argument("--scan-rows", type=int, default=1_000_000)
    ap.add_argument("--scan-queries", type=int, default=1024)
    ap.add_argument("--cpu-sample-tokens", type=int, default=32768)
    ap.add_argument("--scan-cpu-rows", type=int, default=20000,
                    help="rows of the store the CPU baseline of the scan searches (all queries)")
    ap.add_argument("--torch-baseline-steps", type=int, default=40,
                    help="batches the stock-PyTorch op sequence is timed on, on this GPU")
    ap.add_argument("--llama-only", action="store_true", help="run the Llama-shaped leg alone and print its entry")
    ap.add_argument("--per-token-only", action="store_true", help="run the per-token collection leg alone")
    ap.add_argument("--config1-only", action="store_true", help="run configs[0] (GPU and CPU in full) alone")
    ap.add_argument("--adam-only", action="store_true",
                    help="run the per-token Adam leg alone and print its entry (for counter runs on that kernel)")
    ap.add_argument("--plain-loop", action="store_true",
                    help="time the reference's loop shape (forward, backward, hooks, one batch at a time) instead "
                         "of the overlapped loop that CollectorComputer runs by default")
    ap.add_argument("--kernels-only", action="store_true",
                    help="leave out the legs that add no kernel of this library to a counter run: the stock-PyTorch "
                         "baseline, configs[0], configs[3] end to end and the CPU baselines")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy (reads 1 GiB, writes 1 GiB): the known-size "
                         "kernel that hardware byte counters are scaled by")
    return ap.parse_args()


def collection_leg(args, torch, device):
    import bergson_amd as B
    from bergson_amd import ops
    from bergson_amd.collector import CollectorComputer, OverlappedSteps
    from bergson_amd.synthetic import ListDataset, adafactor_moments, lognormal_lengths, make_gpt_neox, random_docs

    lengths = lognormal_lengths(args.docs, seed=0)
    docs = random_docs(lengths, seed=0)
    data = ListDataset(docs)
    batches = B.allocate_batches(lengths, args.token_batch_size)
    need = args.warmup + args.steps
    if len(batches) < need:
        raise SystemExit(f"{len(batches)} batches < warmup + steps = {need}: lower --steps or raise --docs")
    model = make_gpt_neox("pythia-160m", torch.bfloat16, device, seed=0)
    moments = adafactor_moments(model.base_model, seed=0)
    normalizers = {n: B.AdafactorNormalizer(row=r.to(device), col=c.to(device)) for n, (r, c) in moments.items()}
    processor = B.GradientProcessor(normalizers=normalizers, projection_dim=16, projection_type="normal")
    run_dir = tempfile.mkdtemp(prefix="bgx_bench_")
    overlap = not args.plain_loop

    def make_collector(tag):
        cfg = B.IndexConfig(run_path=os.path.join(run_dir, tag), projection_dim=16, projection_type="normal",
                            token_batch_size=args.token_batch_size)
        return cfg, B.GradientCollector(model=model.base_model, cfg=cfg, data=data, processor=processor,
                                        store_dtype=torch.float16)

    # untimed: the first W batches through the same entry point
    if args.warmup:
        cfg, collector = make_collector("warmup")
        CollectorComputer(model=model, data=data, collector=collector, batches=batches[:args.warmup], cfg=cfg,
                          overlap_backward=overlap).run_with_collector_hooks()
        del collector
    timed_batches = batches[args.warmup:need]
    tokens = sum(lengths[i] for indices in timed_batches for i in indices)

    # timed: run_with_collector_hooks over the K batches, padding / upload / flush / teardown included
    cfg, collector = make_collector("store")
    computer = CollectorComputer(model=model, data=data, collector=collector, batches=timed_batches, cfg=cfg,
                                 overlap_backward=overlap)
    torch.cuda.synchronize()
    ops.collect_timer = []
    ops.collect_timing_start(args.steps + 8)
    t0 = time.perf_counter()
    computer.run_with_collector_hooks()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    timer, ops.collect_timer = ops.collect_timer, None
    kernel_only_ms = ops.collect_timing_stop()
    store = collector.builder.grad_buffer
    nonzero = int((abs(store[:, :256].astype("float32")).sum(axis=1) > 0).sum())
    total_processed = int(computer.total_processed)
    del collector, computer

    # the same batches once more, padded and uploaded beforehand
    cfg, collector = make_collector("prestaged")
    fwd_bwd = B.fwd_bwd_factory(cfg)
    staged = []
    for indices in timed_batches:
        b = data[indices]
        x, y, _, mask = B.pad_and_tensor(b["input_ids"], device=device, sync_max_len=False)
        staged.append((indices, b, x, y, mask))
    padded = sum(int(item[2].numel()) for item in staged)
    overlapped = OverlappedSteps(model, collector, cfg) if overlap else None
    torch.cuda.synchronize()
    p0 = time.perf_counter()
    for indices, b, x, y, mask in staged:
        if overlapped is not None:
            overlapped.step(indices, b, x, y, mask)
            continue
        with collector.with_batch(mask):
            losses = fwd_bwd(model, x, y, b)
        collector.process_batch(indices, losses=losses)
    if overlapped is not None:
        overlapped.drain()
    collector.builder.flush()
    torch.cuda.synchronize()
    p1 = time.perf_counter()
    if overlapped is not None:
        n_streams = overlapped._n_streams
        overlapped.close()
    collector.remove_hooks()

    bracket_ms = sum(e0.elapsed_time(e1) for e0, e1, _ in timer)
    kernel_ms = sum(kernel_only_ms)
    assert len(kernel_only_ms) == len(timer) == len(timed_batches), (len(kernel_only_ms), len(timer))
    kernel_bytes = sum(nb for _, _, nb in timer)
    achieved = kernel_bytes / (kernel_ms * 1e-3) / 1e9 if kernel_ms > 0 else 0.0
    out = {
        "seconds": t1 - t0,
        "tokens": tokens,
        "padded_tokens": padded,
        "total_processed": total_processed,
        "prestaged_seconds": p1 - p0,
        "launches": len(timer),
        "kernel_ms_per_launch": kernel_ms / max(1, len(timer)),
        "bracket_ms_per_launch": bracket_ms / max(1, len(timer)),
        "kernel_bytes_per_launch": kernel_bytes / max(1, len(timer)),
        "achieved_gbs": achieved,
        "n_batches_total": len(batches),
        "store_rows_nonzero": nonzero,
        "total_tokens_all_docs": int(sum(lengths)),
        "loop": "plain (one batch at a time)" if not overlap else
                f"overlapped (backward pass of batch i beside the forward pass of batch i+1, batches alternating "
                f"between {n_streams} streams, the collection launch alone on the GPU)",
    }
    extra = {"model": model, "moments": moments, "batches": batches, "data": data}
    del collector
    return out, docs, lengths, extra


def gpu_torch_baseline_leg(args, torch, device, docs, lengths, extra):
    """The reference's hook sequence issued as stock PyTorch ops on this GPU, on the first batches after the
    warm-up ones of the same workload: what the fused launch replaces (module forward and full-backward hooks,
    a * rsqrt(col), a @ R^T, g * factor, g @ L^T, g^T a, clamp, cat, scatter into the store)."""
    from oracle import hooks as ohooks
    from oracle import loop as oloop

    model, batches = extra["model"], extra["batches"]
    norms = {n: ohooks.Adafactor(row=r.to(device), col=c.to(device)) for n, (r, c) in extra["moments"].items()}
    warm = batches[:3]
    timed = batches[args.warmup:args.warmup + args.torch_baseline_steps]
    oloop.collect(model, model.base_model, docs, warm, p=16, normalizers=norms, save_dtype=torch.float16, device=device)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    oloop.collect(model, model.base_model, docs, timed, p=16, normalizers=norms, save_dtype=torch.float16,
                  device=device)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    tok = sum(lengths[i] for b in timed for i in b)
    return {"value": tok / dt, "unit": "tokens/s", "ms_per_step": dt / len(timed) * 1e3, "steps": len(timed),
            "what": "reference op sequence (PyTorch-ROCm ops from module hooks, one batch at a time, rows kept on the "
                    "device) on the same model, batches and GPU"}


class BoardPower:
    """Samples the board's power sensor (hwmon `power1_input`, microwatts) every 20 ms while the block runs.

    The matrix-bound kernels run the chip into its power limit (`power1_cap`), which is what sets their clocks:
    the legs that time them report the power they drew beside their rate.  `report()` is None where the sensor
    cannot be read."""

    def __init__(self):
        import glob
        import threading

        found = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input"))
        self.path = found[0] if found else None
        self.samples: list[float] = []
        self._stop = threading.Event()
        self._thread = threading.Thread(target=self._run, daemon=True)

    def _read(self, path):
        try:
            with open(path) as f:
                return int(f.read()) / 1e6
        except (OSError, ValueError):
            return None

    def _run(self):
        while not self._stop.is_set():
            w = self._read(self.path)
            if w is not None:
                self.samples.append(w)
            self._stop.wait(0.02)

    def __enter__(self):
        if self.path is not None:
            self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        if self.path is not None:
            self._thread.join()

    def report(self):
        if not self.samples:
            return None
        cap = self._read(self.path.replace("power1_input", "power1_cap"))
        return {"mean_w": sum(self.samples) / len(self.samples), "max_w": max(self.samples), "cap_w": cap,
                "samples": len(self.samples)}


def scan_leg(args, torch, device):
    from bergson_amd import ops

    n, D, Q, k = args.scan_rows, 12288, args.scan_queries, 100
    gen = torch.Generator(device=device).manual_seed(1)
    store = torch.empty((n, D), dtype=torch.float16, device=device)
    step = 65536
    for lo in range(0, n, step):
        hi = min(n, lo + step)
        blk = torch.randn((hi - lo, D), generator=gen, device=device)
        heavy = torch.rand((hi - lo, 1), generator=gen, device=device) < 0.05
        store[lo:hi] = (blk * torch.where(heavy, 10.0, 1.0)).to(torch.float16)
    q = torch.randn((Q, D), generator=gen, device=device)
    q = q / q.norm(dim=1, keepdim=True)
    qd = (q * 64.0).to(torch.float16)

    def run():
        # per-query top-k, and per row the max and the mean over the queries, in one pass over the store
        return ops.scan(store, qd, unit_norm=True, k=k, query_scale=1.0 / 64.0, want_row_max=True,
                        want_row_mean=True)

    # warm-up; it also hands out the row sums of squares that the known-norms scan below is given
    sumsq = ops.scan(store, qd, unit_norm=True, k=k, query_scale=1.0 / 64.0, want_row_max=True, want_row_mean=True,
                     want_sumsq=True).sumsq
    torch.cuda.synchronize()
    reps = 10  # the first scans of a burst run ~1 % slower (the chip's clocks settle under sustained load)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with BoardPower() as power:
        e0.record()
        for _ in range(reps):
            res = run()
        e1.record()
        torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / reps
    flops = 2.0 * n * D * Q
    out = {
        "rows": n, "dim": D, "queries": Q, "k": k, "ms": ms, "rows_per_s": n / (ms * 1e-3),
        "roofline": {"bound": "mfma", "achieved": flops / (ms * 1e-3) / 1e12, "peak": MFMA_F16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": flops / (ms * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS,
                     "traffic": n * D * 2 * SCAN_TRAFFIC_RATIO_Q1024,
                     "kernel": "bgx::scan_wide_kernel<f16_t> (384 x 256 tiles, operands loaded straight into LDS)"},
        "hbm_gbs": n * D * 2 / (ms * 1e-3) / 1e9,
        "top1_mean": float(res.topk_values[:Q, 0].mean().item()),
        "board_power": power.report(),
    }
    # the same scan with the store's row norms known from an earlier scan, as Attributor runs every search after
    # its first (the reference normalises an index once, when it loads it): the tile kernel's K loop without the
    # sums of squares
    def run_known():
        return ops.scan(store, qd, unit_norm=True, k=k, query_scale=1.0 / 64.0, want_row_max=True,
                        want_row_mean=True, row_sumsq=sumsq)

    res_known = run_known()
    torch.cuda.synchronize()
    with BoardPower() as power:
        e0.record()
        for _ in range(reps):
            run_known()
        e1.record()
        torch.cuda.synchronize()
    ms_known = e0.elapsed_time(e1) / reps
    out["known_row_norms"] = {
        "ms": ms_known, "rows_per_s": n / (ms_known * 1e-3),
        "roofline": {"bound": "mfma", "achieved": flops / (ms_known * 1e-3) / 1e12, "peak": MFMA_F16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": flops / (ms_known * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS},
        "same_top_k": bool(torch.equal(res_known.topk_indices, res.topk_indices)),
        "board_power": power.report(),
        "what": "bgx_scan_known_norms: row sums of squares taken from an earlier scan of the store instead of "
                "being summed again in the K loop",
    }
    # for scale: the library's GEMM (hipBLASLt through torch.matmul) on the scan's shape -- scores only, no norms,
    # no selection; 2 GB of fp16 scores written.  Both run the chip into its power limit, which sets the clocks.
    dense = torch.empty((n, Q), dtype=torch.float16, device=device)
    qt = qd.T  # a view: both operands contiguous along D, the layout the library is fastest on
    torch.matmul(store, qt, out=dense)
    torch.cuda.synchronize()
    with BoardPower() as power:
        e0.record()
        for _ in range(reps):
            torch.matmul(store, qt, out=dense)
        e1.record()
        torch.cuda.synchronize()
    ms_lib = e0.elapsed_time(e1) / reps
    out["library_gemm_same_shape"] = {"ms": ms_lib, "tflops": flops / (ms_lib * 1e-3) / 1e12,
                                      "frac_of_peak": flops / (ms_lib * 1e-3) / 1e12 / MFMA_F16_PEAK_TFLOPS,
                                      "board_power": power.report(),
                                      "what": "torch.matmul(store [n, D] fp16, queries^T [D, Q]) -> [n, Q] fp16"}
    del dense, qt
    # the one pass that forms those sums when an index is loaded (Attributor: the reference normalises the index
    # at load time), bit-equal to the sums the scan hands out
    loaded = ops.row_sumsq(store)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(reps):
        ops.row_sumsq(store)
    e1.record()
    torch.cuda.synchronize()
    ms_norms = e0.elapsed_time(e1) / reps
    out["row_norms_at_load"] = {
        "ms": ms_norms, "equal_to_the_scans_own_sums": bool(torch.equal(loaded, sumsq)),
        "roofline": {"bound": "hbm", "achieved": n * D * 2 / (ms_norms * 1e-3) / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": n * D * 2 / (ms_norms * 1e-3) / 1e9 / HBM_PEAK_GBS, "kernel": "bgx::row_sumsq_kernel<f16_t, true>"}}
    del sumsq, res_known, loaded
    # the HBM-bound regime: few queries per pass (the streaming kernel, one block of 16 queries or two)
    for nq in (32, 8):
        qs = qd[:nq].contiguous()
        ops.scan(store, qs, unit_norm=True, k=k, query_scale=1.0 / 64.0)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            ops.scan(store, qs, unit_norm=True, k=k, query_scale=1.0 / 64.0)
        e1.record()
        torch.cuda.synchronize()
        ms_few = e0.elapsed_time(e1) / reps
        gbs = n * D * 2 / (ms_few * 1e-3) / 1e9
        out[f"q{nq}"] = {"ms": ms_few, "rows_per_s": n / (ms_few * 1e-3),
                         "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                      "frac": gbs / HBM_PEAK_GBS, "traffic": n * D * 2 * SCAN_TRAFFIC_RATIO_FEW}}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = scan_cpu_baseline(args, torch, store, qd, k)
    del store
    torch.cuda.empty_cache()
    return out


def scan_cpu_baseline(args, torch, store, qd, k):
    """The reference's search (bergson/query/attributor.py:169-235: index and queries to fp32, unit norms,
    Q x N score matrix, torch.topk) on the host cores, on the first rows of the same store."""
    from oracle import scan as oscan

    n = min(args.scan_cpu_rows, store.shape[0])
    rows = store[:n].cpu()
    q = qd.cpu()
    t0 = time.perf_counter()
    vals, idx = oscan.attributor_search({"g": rows}, {"g": q}, ["g"], k, unit_norm=True)
    dt = time.perf_counter() - t0
    return {"value": n / dt, "unit": "rows/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"the first {n} of {store.shape[0]} rows against all {q.shape[0]} queries, top-{k}, in {dt:.2f} s; the "
                      f"scan is linear in the rows, so the whole store would take {store.shape[0] / n:.0f} x as long"}


def per_token_leg(args, torch, device):
    """configs[1]'s 48 modules with one row per token (attribute_tokens) at p = 16: the persistent collection kernel
    writing every valid token's p x p blocks, 2 x 2048 tokens per launch, bf16 rows.  Kernel only, synthetic a / g."""
    from bergson_amd import ops

    N, S, p, d = 2, 2048, 16, 768
    gen = torch.Generator(device=device).manual_seed(3)
    rnd = lambda *shape: torch.randn(*shape, generator=gen, device=device)
    mods, col = [], 0
    for layer in range(12):
        for I, O in ((d, 3 * d), (d, d), (d, 4 * d), (4 * d, d)):
            rs, cs = ops.adafactor_scales(rnd(O).abs() * 1e-4 + 1e-12, rnd(I).abs() * 1e-4 + 1e-12, torch.bfloat16)
            mods.append(ops.ModuleInput(a=rnd(N, S, I).to(torch.bfloat16), g=(rnd(N, S, O) * 0.01).to(torch.bfloat16),
                                        r_in=(rnd(p, I) / 4).to(torch.bfloat16), r_out=(rnd(p, O) / 4).to(torch.bfloat16),
                                        out_col=col, col_scale=cs, row_scale=rs))
            col += p * p
    lengths = torch.full((N,), S, dtype=torch.int32, device=device)
    offsets = torch.arange(N, device=device, dtype=torch.int64) * (S - 1)
    out = torch.zeros(N * (S - 1), col, device=device, dtype=torch.bfloat16)
    reps = 10
    ops.collect_tok(mods, p, out, lengths=lengths, row_offsets=offsets, lo=-3e38, hi=3e38)
    torch.cuda.synchronize()
    ops.collect_timing_start(reps)
    for _ in range(reps):
        ops.collect_tok(mods, p, out, lengths=lengths, row_offsets=offsets, lo=-3e38, hi=3e38)
    torch.cuda.synchronize()
    ms = ops.collect_timing_stop()
    ms = sum(ms) / len(ms)
    read = N * S * sum(m.a.shape[2] + m.g.shape[2] for m in mods) * 2
    written = out.numel() * 2
    gbs = (read + written) / (ms * 1e-3) / 1e9
    return {"workload": "configs[1] modules, per-token rows: 48 Pythia-160m modules, 2 x 2048 tokens, p=16, Adafactor, "
                        "bf16 rows of 12288",
            "ms_per_launch": ms, "tokens_per_s_hooks_only": N * S / (ms * 1e-3),
            "roofline": {"bound": "hbm", "kernel": "bgx::collect_persist_kernel<bf16_t, true, 2, 4, true, false, 1, false> (every token's "
                                                  "projections, written contiguously) + bgx::token_rows_kernel (whole store "
                                                  "rows from them), one event pair around both",
                         "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                         "bytes_read": read, "bytes_written": written,
                         "traffic": (read + written) * PER_TOKEN_TRAFFIC_RATIO}}


def wide_projection_leg(args, torch, device):
    """configs[1]'s 48 modules at projection dimensions above 16: the streamed collection kernel with two (p = 32)
    or four (p = 64) blocks of 16 projection columns per k-step, fragments from the table in global memory, 4 x 1024
    tokens per launch; per-sequence rows, and per-token rows (at p = 32; in two steps, bf16 rows of 49 152 values).
    Kernel only, synthetic a / g; the event pair spans the collection kernel (and, per token, the kernel that writes
    the rows), not the table's preparation before it nor the sum of the tiles' partial blocks behind it."""
    from bergson_amd import _lib, ops

    N, S, d = 4, 1024, 768
    gen = torch.Generator(device=device).manual_seed(4)
    rnd = lambda *shape: torch.randn(*shape, generator=gen, device=device)
    shapes = [(d, 3 * d), (d, d), (d, 4 * d), (4 * d, d)] * 12
    acts = [(rnd(N, S, I).to(torch.bfloat16), (rnd(N, S, O) * 0.01).to(torch.bfloat16)) for I, O in shapes]
    lengths = torch.full((N,), S, dtype=torch.int32, device=device)
    read = N * S * sum(I + O for I, O in shapes) * 2
    out = {"workload": "configs[1] modules, per-sequence rows at p = 32 and 64: 48 Pythia-160m modules, 4 x 1024 "
                       "tokens, Adafactor, fp16 rows", "bytes_read": read}
    reps = 10
    for p in (32, 64):
        mods, col = [], 0
        for (I, O), (a, g) in zip(shapes, acts):
            rs, cs = ops.adafactor_scales(rnd(O).abs() * 1e-4 + 1e-12, rnd(I).abs() * 1e-4 + 1e-12, torch.bfloat16)
            mods.append(ops.ModuleInput(a=a, g=g, r_in=(rnd(p, I) / 4).to(torch.bfloat16),
                                        r_out=(rnd(p, O) / 4).to(torch.bfloat16), out_col=col, col_scale=cs, row_scale=rs))
            col += p * p
        rows = torch.zeros(N, col, device=device, dtype=torch.float16)
        ops.collect_seq(mods, p, rows, lengths=lengths, lo=-6e4, hi=6e4)
        torch.cuda.synchronize()
        ops.collect_timing_start(reps)
        for _ in range(reps):
            ops.collect_seq(mods, p, rows, lengths=lengths, lo=-6e4, hi=6e4)
        torch.cuda.synchronize()
        ms = ops.collect_timing_stop()
        ms = sum(ms) / len(ms)
        gbs = read / (ms * 1e-3) / 1e9
        out[f"p{p}"] = {"ms_per_launch": ms, "kernel": _lib.last_kernel(_lib.FAMILY_COLLECT),
                        "tokens_per_s_hooks_only": N * S / (ms * 1e-3),
                        "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                     "frac": gbs / HBM_PEAK_GBS, "traffic": read * WIDE_TRAFFIC_RATIO[p]}}
        if p == 32:
            offsets = torch.arange(N, device=device, dtype=torch.int64) * (S - 1)
            tok_rows = torch.zeros(N * (S - 1), col, device=device, dtype=torch.bfloat16)
            run = lambda: ops.collect_tok(mods, p, tok_rows, lengths=lengths, row_offsets=offsets, lo=-3e38, hi=3e38)
            run()
            torch.cuda.synchronize()
            ops.collect_timing_start(reps)
            for _ in range(reps):
                run()
            torch.cuda.synchronize()
            ms = ops.collect_timing_stop()
            ms = sum(ms) / len(ms)
            written = tok_rows.numel() * 2
            gbs = (read + written) / (ms * 1e-3) / 1e9
            out["p32_per_token"] = {"ms_per_launch": ms, "kernel": _lib.last_kernel(_lib.FAMILY_COLLECT),
                                    "bytes_written": written,
                                    "roofline": {"bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                                 "frac": gbs / HBM_PEAK_GBS,
                                                 "traffic": (read + written) * WIDE_TOK_TRAFFIC_RATIO}}
            del tok_rows
        del mods, rows
    return out


def llama_leg(args, torch, device):
    """configs[4]'s module shapes through a model: four layers of a Llama-3-8B-shaped decoder (28 hooked modules
    of 4096 x {4096, 1024, 14336}), batches of 2 x 2048 tokens, p = 16, Adafactor, fp16 store.  The roofline entry
    is the collection kernel of those launches (the streamed kernel with its projection fragments in a global
    table, since 4096 x 14336 does not fit on chip), timed by event pairs on its stream."""
    import bergson_amd as B
    from bergson_amd import ops
    from bergson_amd.collector import CollectorComputer
    from bergson_amd.synthetic import ListDataset, adafactor_moments, make_llama, random_docs

    layers, n_batches, warm = 4, 6, 2
    lengths = [2048] * (2 * (n_batches + warm))
    docs = random_docs(lengths, vocab=128256, seed=5)
    data = ListDataset(docs)
    batches = [[2 * i, 2 * i + 1] for i in range(n_batches + warm)]
    model = make_llama(torch.bfloat16, device, layers=layers, seed=0)
    moments = adafactor_moments(model.base_model, seed=0)
    normalizers = {n: B.AdafactorNormalizer(row=r.to(device), col=c.to(device)) for n, (r, c) in moments.items()}
    processor = B.GradientProcessor(normalizers=normalizers, projection_dim=16, projection_type="normal")
    cfg = B.IndexConfig(run_path="", projection_dim=16, projection_type="normal", token_batch_size=4096)

    def run(which):
        col = B.GradientCollector(model=model.base_model, cfg=cfg, data=data, processor=processor,
                                  store_dtype=torch.float16)
        CollectorComputer(model=model, data=data, collector=col, batches=which, cfg=cfg).run_with_collector_hooks()
        torch.cuda.synchronize()
        return col

    run(batches[:warm])
    ops.collect_timer = []
    ops.collect_timing_start(n_batches + 2)
    t0 = time.perf_counter()
    col = run(batches[warm:])
    dt = time.perf_counter() - t0
    timer, ops.collect_timer = ops.collect_timer, None
    ms = ops.collect_timing_stop()
    assert len(ms) == n_batches, len(ms)
    nbytes = sum(nb for _, _, nb in timer) / len(timer)
    ms_launch = sum(ms) / len(ms)
    gbs = nbytes / (ms_launch * 1e-3) / 1e9
    rows = col.builder.grad_buffer
    assert rows.shape[1] == 7 * layers * 256
    out = {"workload": f"configs[4] shapes: {layers} layers of a Llama-3-8B-shaped decoder (28 modules), 2 x 2048-token "
                       "batches, p=16, Adafactor, fp16 store",
           "tokens_per_s_this_4_layer_model": 4096 * n_batches / dt, "ms_per_step": dt / n_batches * 1e3,
           "roofline": {"bound": "hbm", "kernel": "bgx::collect_persist_kernel<bf16_t, false, 2, 4, true, true, 1, false> "
                                                  "(streamed loads, projection fragments from a global table, shared by the workgroup through LDS)",
                        "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                        "bytes_per_launch": nbytes, "ms_per_launch": ms_launch, "launches": len(ms),
                        "ms_per_launch_with_table_build_and_finalize":
                            sum(e0.elapsed_time(e1) for e0, e1, _ in timer) / len(timer),
                        "traffic": nbytes * LLAMA_TRAFFIC_RATIO}}
    del col, model
    torch.cuda.empty_cache()
    return out


def adam_leg(args, torch, device):
    """Per-token gradients under an Adam normalizer at p = 32 (configs[3]: Pythia-410m shape): the four Linear
    modules of one layer on one 4096-token batch, i.e. the fused kernel that dominates that configuration."""
    from bergson_amd import ops

    N, S, p, d = 4, 1024, 32, 1024
    gen = torch.Generator(device=device).manual_seed(2)
    rnd = lambda *shape: torch.randn(*shape, generator=gen, device=device)
    lengths = torch.full((N,), S, dtype=torch.int32, device=device)
    offsets = torch.arange(N, device=device, dtype=torch.int64) * (S - 1)
    # the configuration's store layout: rows of 96 modules x p x p values, a module's block 196 608 bytes further on
    # in every row (the four modules timed here write blocks 40..43)
    n_blocks = 96
    out = torch.zeros(N * (S - 1), n_blocks * p * p, device=device, dtype=torch.bfloat16)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    # 30 timed launches behind 5 untimed ones per module: the first launches of a burst run at lower clocks (5 timed
    # launches read 7 % slower than 60), and the configuration this stands for issues 96 of them per batch
    reps, total_ms, total_flops, modules = 30, 0.0, 0.0, {}
    power = BoardPower()
    power.__enter__()
    for block, (name, (I, O)) in enumerate((("query_key_value", (d, 3 * d)), ("dense", (d, d)),
                                            ("dense_h_to_4h", (d, 4 * d)), ("dense_4h_to_h", (4 * d, d)))):
        a = rnd(N, S, I).to(torch.bfloat16)
        g = (rnd(N, S, O) * 0.01).to(torch.bfloat16)
        v = torch.rand(O, I, generator=gen, device=device) * 1e-5 + 1e-10
        prep = ops.AdamPrepared(rnd(p, I).to(torch.bfloat16), rnd(p, O).to(torch.bfloat16), v, (40 + block) * p * p)
        run = lambda: ops.collect_adam(prep, a, g, out, per_token=True, lengths=lengths, rows=offsets, lo=-3e38,
                                       hi=3e38)
        for _ in range(5):
            run()
        torch.cuda.synchronize()
        e0.record()
        for _ in range(reps):
            run()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        flops = 2.0 * N * S * I * O * p
        modules[name] = {"I": I, "O": O, "ms": ms, "tflops": flops / (ms * 1e-3) / 1e12}
        total_ms += ms
        total_flops += flops
        del a, g, v, prep
    power.__exit__()
    tf = total_flops / (total_ms * 1e-3) / 1e12
    del out
    torch.cuda.empty_cache()
    return {"workload": "configs[3]: one Pythia-410m layer, 4 x 1024 tokens, p=32, Adam, per-token rows (bf16) "
                        "written as blocks of the configuration's 98 304-wide store rows",
            "end_to_end": None if args.kernels_only else adam_end_to_end(torch, device),
            "ms_per_layer": total_ms, "tokens_per_s_24_layers_hooks_only": N * S / (total_ms * 24e-3),
            "board_power": power.report(),
            "roofline": {"bound": "mfma", "achieved": tf, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": tf / MFMA_F16_PEAK_TFLOPS, "traffic": ADAM_TRAFFIC_BYTES_PER_LAYER,
                         "kernel": "bgx::adam_fused_wide_kernel<bf16_t>"},
            "modules": modules}


def adam_end_to_end(torch, device, n_batches=8, warm=2):
    """configs[3] through the product loop on a slice: a Pythia-410m-shaped model (24 layers, 96 hooked modules),
    documents of 1024 tokens in batches of 4, p = 32, Adam second moments |N(0,1)| * 1e-5 for every module, per-token
    rows of 98 304 bf16 values written into the device-resident store (`warm` untimed batches first, in which the
    Adam tables are built)."""
    import bergson_amd as B
    from bergson_amd.collector import CollectorComputer
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs

    p, per_batch, S = 32, 4, 1024
    lengths = [S] * (per_batch * (n_batches + warm))
    data = ListDataset(random_docs(lengths, seed=4))
    batches = [list(range(per_batch * i, per_batch * (i + 1))) for i in range(n_batches + warm)]
    model = make_gpt_neox("pythia-410m", torch.bfloat16, device, seed=0)
    gen = torch.Generator(device=device).manual_seed(3)
    normalizers = {}
    for name, mod in model.base_model.named_modules():
        if isinstance(mod, torch.nn.Linear):
            v = torch.randn(mod.out_features, mod.in_features, generator=gen, device=device).abs_() * 1e-5
            normalizers[name] = B.AdamNormalizer(weight_avg_sq=v)
    processor = B.GradientProcessor(normalizers=normalizers, projection_dim=p, projection_type="normal")
    cfg = B.IndexConfig(run_path="", projection_dim=p, projection_type="normal", token_batch_size=per_batch * S,
                        attribute_tokens=True)

    from bergson_amd.collector import OverlappedSteps

    staged = []
    for indices in batches:
        b = data[indices]
        x, y, _, mask = B.pad_and_tensor(b["input_ids"], device=device, sync_max_len=False)
        staged.append((indices, b, x, y, mask))
    col = B.GradientCollector(model=model.base_model, cfg=cfg, data=data, processor=processor)
    steps = OverlappedSteps(model, col, cfg)
    for item in staged[:warm]:
        steps.step(*item)
    steps.drain()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for item in staged[warm:]:
        steps.step(*item)
    steps.drain()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    steps.close()
    device_resident = bool(col.builder.direct)
    f0 = time.perf_counter()
    col.builder.flush()
    torch.cuda.synchronize()
    flush_s = time.perf_counter() - f0
    col.remove_hooks()
    rows, width = col.builder.grad_buffer.shape
    filled = int((col.builder.grad_buffer[:, 40 * p * p] != 0).sum())
    modules = len(col.target_info)
    del col, steps, model, normalizers, processor, staged
    torch.cuda.empty_cache()
    tokens = n_batches * per_batch * S
    return {"workload": f"configs[3] on a slice: Pythia-410m-shaped GPT-NeoX bf16 ({modules} hooked modules), {n_batches} "
                        f"batches of {per_batch} x {S} tokens after {warm} untimed ones (in which the Adam tables are "
                        f"built), p={p}, Adam normalizer on every module, per-token rows of {width} bf16 values",
            "value": tokens / dt, "unit": "tokens/s", "ms_per_batch": dt / n_batches * 1e3, "batches": n_batches,
            "store_rows": rows, "store_row_width": width, "store_device_resident": device_resident,
            "rows_written": filled,
            "timed_region": "the product loop (OverlappedSteps: forward, backward, 96 fused launches per batch) over the "
                            "timed batches, token ids already on the device, rows landing in the device-resident store",
            "flush_seconds": flush_s,
            "flush": f"copying the {rows * width * 2 / 1e9:.1f} GB store to host memory afterwards (once per job)"}


def config1_leg(args, torch, device):
    """configs[0] in full, the one configuration the reference's CPU path runs: Pythia-14m-shaped fp32 model, 64
    documents of 256 uniform-random tokens, 2048-token batches, p = 16 on the 24 Linear modules, no normalizer,
    per-sequence rows -- the product loop on the GPU (second pass over the data in this process) beside the
    oracle's loop on the host cores, both over all 16 384 tokens, and their rows compared."""
    import numpy as np

    import bergson_amd as B
    from bergson_amd.collector import CollectorComputer
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs
    from oracle import loop as oloop

    lengths = [256] * 64
    docs = random_docs(lengths, seed=0)
    data = ListDataset(docs)
    batches = B.allocate_batches(lengths, 2048)
    tokens = sum(lengths)
    gpu = make_gpt_neox("pythia-14m", torch.float32, device, seed=0)
    cfg = B.IndexConfig(run_path="", projection_dim=16, projection_type="normal", token_batch_size=2048)
    processor = B.GradientProcessor(projection_dim=16, projection_type="normal")

    def run():
        col = B.GradientCollector(model=gpu.base_model, cfg=cfg, data=data, processor=processor)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        CollectorComputer(model=gpu, data=data, collector=col, batches=batches, cfg=cfg).run_with_collector_hooks()
        torch.cuda.synchronize()
        return time.perf_counter() - t0, col

    run()
    dt, col = run()
    got = torch.from_numpy(np.array(col.builder.grad_buffer))
    out = {"workload": "configs[0]: Pythia-14m-shaped GPT-NeoX fp32, 64 x 256 tokens, 2048-token batches, p=16 normal "
                       "projections on 24 modules, no normalizer, per-sequence rows",
           "value": tokens / dt, "unit": "tokens/s", "seconds": dt, "tokens": tokens, "batches": len(batches),
           "dtype": "f32"}
    if not args.no_cpu_baseline:
        cpu = make_gpt_neox("pythia-14m", torch.float32, "cpu", seed=0)
        t0 = time.perf_counter()
        want, _ = oloop.collect(cpu, cpu.base_model, docs, batches, p=16)
        cdt = time.perf_counter() - t0
        err = ((got.double() - want.double()).norm() / want.double().norm()).item()
        out["cpu_baseline"] = {"value": tokens / cdt, "unit": "tokens/s", "cores": torch.get_num_threads(),
                               "kind": "port", "seconds": cdt,
                               "sample": f"the whole configuration: {tokens} tokens in {cdt:.1f} s (reference op "
                                         "sequence on PyTorch CPU, fp32)"}
        out["rel_l2_gpu_vs_cpu_rows"] = err
    return out


def cpu_baseline_leg(args, torch, docs, lengths):
    """The CPU oracle on the first documents of the same workload, about `cpu_sample_tokens` tokens."""
    from bergson_amd.synthetic import adafactor_moments, make_gpt_neox
    from oracle import hooks as ohooks
    from oracle import loop as oloop

    picked, tok = [], 0
    for i, l in enumerate(lengths):
        if tok + l > args.cpu_sample_tokens and picked:
            break
        picked.append(i)
        tok += l
    sub_docs = [docs[i] for i in picked]
    sub_len = [lengths[i] for i in picked]
    batches = oloop.allocate_batches(sub_len, args.token_batch_size)
    model = make_gpt_neox("pythia-160m", torch.bfloat16, "cpu", seed=0)
    moments = adafactor_moments(model.base_model, seed=0)
    norms = {n: ohooks.Adafactor(row=r, col=c) for n, (r, c) in moments.items()}
    t0 = time.perf_counter()
    rows, _ = oloop.collect(model, model.base_model, sub_docs, batches, p=16, normalizers=norms,
                            save_dtype=torch.float16)
    dt = time.perf_counter() - t0
    return {"value": tok / dt, "unit": "tokens/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"{len(picked)} documents / {tok} tokens of the same workload in {dt:.1f} s "
                      f"(reference op sequence on PyTorch CPU, bf16 model, fp16 rows)"}


def end_child_processes() -> list[str]:
    """Names of the child processes this script still had when it was done (worker pools of the libraries it
    used); they are ended, so that nothing outlives the benchmark."""
    import multiprocessing

    import psutil

    names = []
    for child in multiprocessing.active_children():
        child.terminate()
    for child in psutil.Process().children(recursive=True):
        try:
            names.append(" ".join(child.cmdline()[:3]) or child.name())
            child.terminate()
        except psutil.Error:
            pass
    return names


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported in this build "
              "(collection shards by documents with no exchange; the scan shards by store rows)", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU path)", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    import datasets

    datasets.disable_progress_bars()  # the loop's teardown saves a dataset; keep stderr to what this script says

    if args.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.float32, device=device)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()
    if args.scan_only:
        print(json.dumps({"store_scan": scan_leg(args, torch, device)}))
        return
    if args.adam_only:
        print(json.dumps({"adam_per_token": adam_leg(args, torch, device)}))
        return
    if args.llama_only:
        print(json.dumps({"llama8b_layers": llama_leg(args, torch, device)}))
        return
    if args.config1_only:
        print(json.dumps({"config1": config1_leg(args, torch, device)}))
        return
    if args.per_token_only:
        print(json.dumps({"per_token": per_token_leg(args, torch, device)}))
        return
    if args.kernels_only:
        args.no_cpu_baseline = True
    coll, docs, lengths, extra = collection_leg(args, torch, device)
    gpu_torch = None if args.no_scan or args.kernels_only else gpu_torch_baseline_leg(args, torch, device, docs, lengths,
                                                                                     extra)
    del extra
    torch.cuda.empty_cache()
    scan = None if args.no_scan else scan_leg(args, torch, device)
    per_token = None if args.no_scan else per_token_leg(args, torch, device)
    wide = None if args.no_scan else wide_projection_leg(args, torch, device)
    llama = None if args.no_scan else llama_leg(args, torch, device)
    adam = None if args.no_scan else adam_leg(args, torch, device)
    config1 = None if args.no_scan or args.kernels_only else config1_leg(args, torch, device)
    cpu = None if args.no_cpu_baseline else cpu_baseline_leg(args, torch, docs, lengths)

    value = coll["tokens"] / coll["seconds"]
    line = {
        "metric": "grad-collection tokens/sec (Pythia-160m shape, p=16)",
        "value": value,
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": coll["seconds"] / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "configs[1]: Pythia-160m-shaped GPT-NeoX bf16, lognormal(6,1) lengths in [16,2048], "
                        "4096-token batches, p=16 normal projections on 48 modules, Adafactor normalizer, "
                        "per-sequence rows into an fp16 store",
            "documents": args.docs,
            "token_batch_size": args.token_batch_size,
            "tokens_timed": coll["tokens"],
            "padded_tokens_timed": coll["padded_tokens"],
            "total_processed": coll["total_processed"],
            "batches_total": coll["n_batches_total"],
            "loop": coll["loop"],
            "timed_region": "CollectorComputer.run_with_collector_hooks over the timed batches: padding, upload of the "
                            "token ids, forward, backward, fused launch, store flush, teardown artefacts",
            "warm_up_caveat": "in a fresh process the first ~50 batches of new shapes run at ~12 ms instead of ~8.8 (the "
                              "libraries under the model load kernels and pick GEMM variants on first use): with fewer "
                              "than ~50 untimed batches part of that falls into the timed steps and lowers `value`",
        },
        "prestaged": {"value": coll["tokens"] / coll["prestaged_seconds"], "unit": "tokens/s",
                      "ms_per_step": coll["prestaged_seconds"] / args.steps * 1e3,
                      "what": "the same batches once more, padded and uploaded before the clock starts; loop body and "
                              "store flush only"},
        "roofline": {
            "bound": "hbm",
            "kernel": "bgx::collect_persist_kernel<bf16_t, false, 2, 4, true, false, 1, false> and <bf16_t, false, 1, 8, true, false, 1, false> (128- and 64-token tiles, streamed loads, projections in LDS)",
            "achieved": coll["achieved_gbs"],
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": coll["achieved_gbs"] / HBM_PEAK_GBS,
            "traffic": coll["kernel_bytes_per_launch"] * COLLECT_TRAFFIC_RATIO,
            "traffic_source": "bytes_per_launch x 1.036 (rocprofv3 FETCH_SIZE + WRITE_SIZE, profiles/)",
            "bytes_per_launch": coll["kernel_bytes_per_launch"],
            "ms_per_launch": coll["kernel_ms_per_launch"],
            "ms_per_launch_with_descriptor_copy_and_finalize": coll["bracket_ms_per_launch"],
            "launches": coll["launches"],
        },
        "cpu_baseline": cpu,
        "gpu_torch_baseline": gpu_torch,
        "store_scan": scan,
        "per_token": per_token,
        "wide_projection": wide,
        "llama8b_layers": llama,
        "adam_per_token": adam,
        "config1": config1,
    }
    line["child_processes_at_exit"] = end_child_processes()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
