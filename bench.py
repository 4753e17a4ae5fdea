#!/usr/bin/env python3
"""Benchmark of the weight-placement hot path on one MI355X.

A step is one pass of the device-side placement over one batch of synthetic input:
the whole Llama-3-8B bf16 checkpoint (4 safetensors shards, 16.06 GB, seeded) is
resident in HBM as raw file bytes, and one step produces the 195 parameter buffers of
one tensor-parallel rank (TP=8): q/k/v/gate/up sliced by rows and fused into qkv_proj /
gate_up_proj, o/down sliced by columns (strided gather), embedding and lm_head sliced
by vocab, with the per-buffer checksums accumulated in the same kernel.  ``value`` is
placed bytes per second of that step.

Besides the contract line's fields the JSON carries
  roofline      the placement kernel against the HBM roofline (HIP-event time on the
                launch stream, algorithmic bytes = 2 x placed bytes)
  cpu_baseline  the CPU oracle (oracle/, "port" of the reference's CPU path) placing the
                same rank from the same files on this host's cores
  e2e_ingest    the same placement ingested from files (page cache) through the pinned
                ring, against this box's measured pinned host-to-device bandwidth
"""

from __future__ import annotations

import argparse
import json
import os
import shutil
import sys
import tempfile
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0
# HBM bytes per place_kernel launch on the default workload, from the FETCH_SIZE and
# WRITE_SIZE counter runs summarised in profiles/place_kernel_llama3_8b_tp8.txt (each
# counter scaled by its reading for a plain 1 GiB device copy).  Counters cannot be read
# from inside this process, so the figure is carried here and reported only when the
# workload is the profiled one.
PROFILED_TRAFFIC_BYTES = {("llama", 32, 8): 4_095_900_000}


def _log(msg: str) -> None:
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def _pick_workdir(need_bytes: int) -> str | None:
    for base in (os.environ.get("MXP_BENCH_DIR"), "/dev/shm", tempfile.gettempdir()):
        if not base or not os.path.isdir(base):
            continue
        try:
            if shutil.disk_usage(base).free > need_bytes * 1.15:
                return tempfile.mkdtemp(prefix="mxp_bench_", dir=base)
        except OSError:
            continue
    return None


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--rank", type=int, default=3, help="tensor-parallel rank whose slice is placed")
    ap.add_argument("--layers", type=int, default=32, help="reduce only for a quick functional check")
    ap.add_argument("--tile-kib", type=int, default=0, help="destination KiB per workgroup (0 = library default)")
    ap.add_argument("--no-e2e", action="store_true", help="skip the file-ingest leg")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--calibrate", action="store_true",
                    help="also run one plain 1 GiB device copy (a kernel of known traffic, for scaling profiler counters)")
    ap.add_argument("--seed", type=int, default=20240229)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; runs with --gpus above 1 are not part of it "
              "(each rank's placement is independent, so a node's rate is the sum of its ranks').", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the placement path has no CPU fallback", file=sys.stderr)
        return 1
    from modelexpress_amd import _lib, models, synth
    from modelexpress_amd.engine import Checkpoint, PlacementEngine, PlacementPlan

    _lib.lib()  # fail loudly if the HIP library is missing
    tp = 8
    layout = models.Llama(layers=args.layers)
    tensors = layout.checkpoint()
    total_bytes = sum(t.nbytes for t in tensors)
    rv = layout.rank_view(tp_size=tp, tp_rank=args.rank)
    host_threads = min(16, os.cpu_count() or 1)

    want_files = not (args.no_e2e and args.no_cpu)
    workdir = _pick_workdir(total_bytes) if want_files else None
    files_real = workdir is not None
    if workdir is None:
        workdir = tempfile.mkdtemp(prefix="mxp_bench_hdr_")
    try:
        t0 = time.perf_counter()
        if files_real:
            synth.write_checkpoint(tensors, workdir, n_shards=4, seed=args.seed, threads=host_threads)
            _log(f"wrote {total_bytes / 1e9:.2f} GB checkpoint to {workdir} in {time.perf_counter() - t0:.1f}s")
        else:
            synth.write_headers_only(tensors, workdir, n_shards=4)
            _log("no room for checkpoint files: resident leg only")
        ck = Checkpoint(workdir)
        plan = PlacementPlan(ck, rv.params, tp_size=tp, tp_rank=args.rank,
                             stacked_params_mapping=rv.stacked_params_mapping)
        eng = PlacementEngine(0, ring_slots=8, slot_bytes=64 << 20, reader_threads=host_threads, streams=4,
                              tile_bytes=args.tile_kib * 1024)
        totals = plan.totals()
        placed = totals["placed_bytes"]
        algo = totals["kernel_algorithmic_bytes"]
        t0 = time.perf_counter()
        staged = synth.stage_on_device(ck, tensors, seed=args.seed)
        _log(f"staged {sum(int(s.numel()) for s in staged) / 1e9:.2f} GB in HBM in {time.perf_counter() - t0:.1f}s")
        dst = eng.allocate(plan, fill=0)

        if args.calibrate:
            a = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
            b = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
            a.fill_(1)
            b.copy_(a)  # reads 1 GiB, writes 1 GiB
            torch.cuda.synchronize()
            del a, b

        # ---- timed region: exactly K steps, inputs already in HBM ----
        for _ in range(args.warmup):
            eng.execute_resident(plan, staged, dst)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            eng.execute_resident(plan, staged, dst)
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ms_per_step = wall / args.steps * 1e3
        value = placed / (wall / args.steps) / 1e9
        resident_sums = eng.checksums(plan)

        # ---- kernel time: HIP events on the launch stream, one pair per launch ----
        k_ms = []
        info = None
        for _ in range(args.steps):
            info = eng.execute_resident(plan, staged, dst, timed=True)
            k_ms.append(info["kernel_ms"])
        k_avg = sum(k_ms) / len(k_ms)
        achieved = algo / (k_avg * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": round(achieved / HBM_PEAK_GBPS, 4),
                    "traffic": PROFILED_TRAFFIC_BYTES.get(("llama", args.layers, tp)),
                    "kernel": "place_kernel", "kernel_ms_avg": round(k_avg, 4), "kernel_ms_min": round(min(k_ms), 4),
                    "algorithmic_bytes": algo, "workgroups": info["n_workgroups"], "segments": info["n_segments"]}

        out = {
            "metric": "placed-weight GB/s into HBM end-to-end + kernel HBM GB/s vs peak, Llama-3-8B",
            "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": "u8", "data": "synthetic",
            "config": {"workload": "configs[1]: Llama-3-8B-shaped bf16 checkpoint, 4 safetensors shards resident in HBM; "
                                   "one TP=8 rank slice (q/k/v/gate/up rows, o/down columns, vocab-split embeddings), "
                                   "fused QKV and gate_up, 195 buffers with checksums",
                       "layers": args.layers, "tp_size": tp, "tp_rank": args.rank, "checkpoint_bytes": total_bytes,
                       "placed_bytes": placed, "buffers": len(plan.params), "timed": "device placement, one launch per step"},
            "roofline": roofline,
        }

        # ---- end-to-end ingest from files through the pinned ring ----
        agree = True
        if files_real and not args.no_e2e:
            h2d_peak = eng.measure_h2d(256 << 20, 5) / 1e9
            best = None
            for i in range(3):
                dst2 = dst if i else eng.allocate(plan, fill=0)
                st = eng.execute(plan, dst2)
                if i and (best is None or st["wall_seconds"] < best["wall_seconds"]):
                    best = st
            ingest_sums = eng.checksums(plan)
            agree = agree and ingest_sums == resident_sums
            w = best["wall_seconds"]
            out["e2e_ingest"] = {
                "placed_gbps": round(best["placed_bytes"] / w / 1e9, 2), "h2d_gbps": round(best["h2d_bytes"] / w / 1e9, 2),
                "h2d_peak_gbps": round(h2d_peak, 2), "frac_of_h2d_peak": round(best["h2d_bytes"] / w / 1e9 / h2d_peak, 4),
                "wall_s": round(w, 4), "file_bytes": best["file_bytes"], "h2d_bytes": best["h2d_bytes"],
                "reader_threads": host_threads, "ring": "8 x 64 MiB pinned", "source": f"page cache ({workdir})",
                "checksums_match_resident": ingest_sums == resident_sums}
            _log(f"e2e ingest: {out['e2e_ingest']}")

        # ---- CPU baseline: the oracle placing the same rank from the same files ----
        if files_real and not args.no_cpu:
            from oracle import cpu_path

            res = cpu_path.run(workdir, [(p.name, p.dtype, p.shape) for p in rv.params], tp_size=tp, tp_rank=args.rank,
                               stacked=rv.stacked_params_mapping, threads=host_threads, repeats=3)
            cpu_sums = [res["checksums"][p.name] for p in rv.params]
            agree = agree and cpu_sums == resident_sums
            out["cpu_baseline"] = {
                "value": round(res["placed_bytes"] / res["place_s"] / 1e9, 3), "unit": "GB/s", "cores": res["threads"],
                "kind": "port",
                "sample": f"the full TP rank slice ({res['placed_bytes']} placed bytes, {res['n_writes']} writes) from the "
                          f"same files, best of 3; parse {res['parse_s']:.3f}s + plan {res['plan_s']:.3f}s not included",
                "place_s": round(res["place_s"], 4), "host_cpus": os.cpu_count(),
                "checksums_match_gpu": cpu_sums == resident_sums}
        else:
            out["cpu_baseline"] = {"value": None, "unit": "GB/s", "cores": 0, "kind": "port", "sample": "skipped"}
        out["checksums_agree"] = agree
        print(json.dumps(out), flush=True)
        eng.close()
        return 0 if agree else 3
    finally:
        shutil.rmtree(workdir, ignore_errors=True)


if __name__ == "__main__":
    sys.exit(main())
