#!/usr/bin/env python3
"""Benchmark of the MonarchAttention forward pass on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cM] [--T 1]
                    [--variant auto|generic|staged|fused|resident|chained] [--no-cpu] [--no-sdpa] [--no-sweep]
    python bench.py --sweep-n | --sweep-e        # the reference's own sweep protocol, against dense SDPA
    python bench.py --sweep-variants [--T 2] [--head-dim 64] [--sweep-grid class96|fewheads|ragged|mid|short]   # every variant over a grid of shapes: AUTO's choice vs the fastest
    python bench.py --record-traffic FETCH.csv WRITE.csv [--config cM --T 1 --variant auto]

A step is ONE forward call of the hot path (monarch_attention, all T steps)
through the C ABI on synthetic inputs that are already resident in HBM.  The
default workload is the configuration the headline metric is quoted on: fp16,
E=1, H=16, N=4096, D=64, block B=64 (=sqrt(N)), post-pad, no mask, with T=1 as in
the reference's own micro-benchmark protocol (perfbench/bench.py:427-431); T = 1,
2, 3 are reported next to it.  Inputs rotate over enough distinct (q, k, v, out)
sets to exceed the 256 MB Infinity Cache, so every step reads its operands from
HBM.

Prints ONE JSON line.  `value` is the forward throughput in TFLOP/s (matmul
FLOPs on padded sizes, the reference's bmm convention,
experiments/vit/evaluation.py:50-59) over the K timed steps.

`roofline` prices the forward against the 8 TB/s HBM peak: `achieved` is the
COMPULSORY bytes of one forward (read Q, K, V once, write the output once)
divided by the summed average durations of the kernels one forward launches,
each measured with HIP events around back-to-back launches on the launch
stream.  With a one-launch variant that is one kernel and one launch is one
forward; with the per-stage launches the per-kernel figures (which count the
state a stage reads and writes as well) are listed under `stages`, labelled as
including intermediates.  `traffic` is the memory-side bytes one forward moved in
a `rocprofv3 --pmc` run (FETCH_SIZE x 2.00, the factor a plain copy of known size
calibrates, + WRITE_SIZE), read from profiles/traffic.json and only reported when
that file was recorded for the kernel sources as they are now.  `cpu_baseline` is
the CPU oracle (a port of the reference's ma_torch.py) timed on this host.
"""
import argparse
import csv
import hashlib
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "monarch-attention_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

CONFIGS = {  # name: (E, H, N, D, B, T, dtype, scale)  - the benchmark configurations of the reference + the metric configuration
    "cM": (1, 16, 4096, 64, 64, 1, "f16", 1.0),
    "c1": (1, 1, 256, 64, 16, 1, "f32", 1.0),
    "c2": (64, 12, 197, 64, 16, 2, "f16", 0.125),
    "c2b": (64, 12, 256, 64, 16, 2, "f16", 0.125),
    "c3": (16, 12, 512, 64, 32, 2, "bf16", 1.0),
    "c4": (8, 16, 1024, 72, 32, 3, "f16", 1.0),
    "c5": (1, 16, 16384, 64, 128, 3, "f16", 1.0),
    # model shapes beyond those (fp32 goes through the fp32 matrix-core stage kernels)
    "gps": (1, 2, 7600, 48, 128, 2, "f32", 1.0),
    "c3f32": (16, 12, 512, 64, 32, 2, "f32", 1.0),
    "bart": (2, 16, 8192, 64, 64, 2, "bf16", 1.0),
}
HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E peak
MFMA_PEAK_TFLOPS = 2500.0      # dense fp16 / bf16
MFMA_PEAK_TFLOPS_F32 = 157.3   # dense fp32
FETCH_SIZE_FACTOR = 2.00       # FETCH_SIZE under-reports a plain copy of known size by this factor (profiles/traffic_forward_kernels.md)
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "traffic.json")
KERNEL_DIR = os.path.join(ROOT, "monarch-attention_amd", "csrc")
ONE_LAUNCH = ("fused", "resident", "chained")   # variants that are one kernel launch per forward (its name: ma_fwd_kernel_name)


def kernel_source_hash() -> str:
    """Hash of the kernel sources: measured traffic is only quoted for the sources it was measured on."""
    h = hashlib.sha1()
    for name in sorted(os.listdir(KERNEL_DIR)):
        if name.endswith((".h", ".hip")):
            with open(os.path.join(KERNEL_DIR, name), "rb") as f:
                h.update(name.encode())
                h.update(f.read())
    return h.hexdigest()[:16]


def recorded_traffic(config: str, T: int, variant: str):
    """Bytes one forward moved on the memory side according to profiles/traffic.json, or None."""
    try:
        with open(TRAFFIC_JSON) as f:
            db = json.load(f)
    except (OSError, ValueError):
        return None
    e = db.get(f"{config}:T{T}:{variant}")
    if not e or e.get("kernel_source_hash") != kernel_source_hash():
        return None
    return e["bytes_per_forward"]


def record_traffic(args) -> None:
    """Fold two rocprofv3 --pmc counter files (FETCH_SIZE and WRITE_SIZE runs of this script, same
    --config / --T / --variant) into profiles/traffic.json: per forward, the mean KiB per dispatch of
    every forward kernel times the kernels one forward launches."""
    fetch_csv, write_csv = args.record_traffic

    names = ("r_step_mfma", "l_step_mfma", "z_step_mfma", "fused_fwd_mfma", "chain_fwd_mfma", "resident_fwd_mfma", "resident_head_mfma", "resident_head2_mfma",
             "r_step_f32", "l_step_f32", "z_step_f32", "head_fwd_f32", "head_t1_f32")

    def per_kernel(path, counter):
        acc = {}
        with open(path) as f:
            for row in csv.DictReader(f):
                if row["Counter_Name"] != counter:
                    continue
                for short in names:   # mangled or demangled, the kernel's name is in there
                    if short in row["Kernel_Name"]:
                        acc.setdefault(short, []).append(float(row["Counter_Value"]))
        return {k: (sum(v) / len(v), len(v)) for k, v in acc.items()}

    fetch, write = per_kernel(fetch_csv, "FETCH_SIZE"), per_kernel(write_csv, "WRITE_SIZE")
    E, H, N, D, B, T, dt, _ = CONFIGS[args.config]
    T = args.T or T
    # launches of each kernel in one forward (the bench also launches single stages for the per-stage timings:
    # the per-dispatch means make that irrelevant)
    per_fwd = {"r_step_mfma": T, "l_step_mfma": T - 1, "z_step_mfma": 1, "fused_fwd_mfma": 1, "chain_fwd_mfma": 1, "resident_fwd_mfma": 1,
               "resident_head_mfma": 1, "resident_head2_mfma": 1, "r_step_f32": T, "l_step_f32": T - 1, "z_step_f32": 1, "head_fwd_f32": 1, "head_t1_f32": 1}
    kernels, total = {}, 0.0
    for name in sorted(set(fetch) & set(write)):
        rd, wr = fetch[name][0] * 1024 * FETCH_SIZE_FACTOR, write[name][0] * 1024
        n = per_fwd.get(name, 0)
        kernels[name] = {"read_bytes_per_launch": round(rd), "written_bytes_per_launch": round(wr), "launches_per_forward": n,
                         "dispatches_averaged": fetch[name][1]}
        total += n * (rd + wr)
    try:
        with open(TRAFFIC_JSON) as f:
            db = json.load(f)
    except (OSError, ValueError):
        db = {}
    db[f"{args.config}:T{T}:{args.variant}"] = {"bytes_per_forward": round(total), "kernels": kernels,
                                                 "kernel_source_hash": kernel_source_hash(),
                                                 "fetch_size_factor": FETCH_SIZE_FACTOR}
    with open(TRAFFIC_JSON, "w") as f:
        json.dump(db, f, indent=1, sort_keys=True)
        f.write("\n")
    print(json.dumps({"recorded": f"{args.config}:T{T}:{args.variant}", "bytes_per_forward": round(total), "kernels": kernels}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--config", default="cM", choices=sorted(CONFIGS))
    ap.add_argument("--T", type=int, default=None, help="override the number of alternating steps")
    ap.add_argument("--variant", default="auto", choices=["auto", "generic", "staged", "fused", "resident", "chained"])
    ap.add_argument("--rotate-workspaces", action="store_true",
                    help="a workspace per input set (default: all sets share one, like the calls of a model)")
    ap.add_argument("--shared-device", action="store_true",
                    help="do not state that the benchmark owns the GPU (MA_FLAG_DEVICE_EXCLUSIVE): 'auto' then never "
                         "resolves to the fused kernel, as for a caller that shares the device")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sdpa", action="store_true", help="skip the dense SDPA comparison")
    ap.add_argument("--no-sweep", action="store_true", help="skip the T = 1, 2, 3 sweep over the variants")
    ap.add_argument("--sweep-n", action="store_true",
                    help="the reference's sequence-length sweep (perfbench/bench.py:87-127): fp16 E=1 H=12 D=64, N = 2^10..2^14 (and on to 2^16), "
                         "block floor(sqrt(N)), T=1, against dense SDPA")
    ap.add_argument("--sweep-e", action="store_true",
                    help="the reference's batch sweep (perfbench/bench.py:42-85): fp16 N=256 H=12 D=64 block 16, E = 2^3..2^13, T=1")
    ap.add_argument("--sweep-variants", action="store_true",
                    help="what the AUTO policy is judged by: every variant that takes a shape, timed over fp16 shapes of 1 .. 384 heads, "
                         "N = 256 .. 8192, blocks of 16 .. 128 rows (T from --T, default 2; head dim from --head-dim); prints the rows "
                         "and how far AUTO's choice is from the fastest variant")
    ap.add_argument("--head-dim", type=int, default=64, help="head dim of --sweep-variants")
    ap.add_argument("--sweep-grid", default="pow2", choices=["pow2", "class96", "fewheads", "ragged", "mid", "short"],
                    help="shapes of --sweep-variants: power-of-two lengths and blocks, blocks / block counts in the 96-row tile class, "
                         "few heads of thousands of tokens, lengths that are no multiple of the block (197, 500, 1000, 3000, 5000, 7600), "
                         "heads of 256 .. 1000 tokens, or up to thousands of heads of at most 256 tokens")
    ap.add_argument("--sweep-dtype", default="f16", choices=["f16", "bf16", "f32"], help="operand dtype of --sweep-variants")
    ap.add_argument("--sweep-mask", action="store_true", help="--sweep-variants with a key / query mask (int64, ~10 %% of the tokens masked out in whole runs)")
    ap.add_argument("--sweep-pre-pad", action="store_true", help="--sweep-variants with the padding at the front")
    ap.add_argument("--record-traffic", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="fold two rocprofv3 --pmc counter_collection.csv files into profiles/traffic.json (no GPU needed)")
    ap.add_argument("--matrix", action="store_true",
                    help="time ma_matrix (the dense (E,H,N,N) attention matrix of get_matrix) instead of the forward metric")
    ap.add_argument("--backward", action="store_true",
                    help="time ma_bwd (gradients of q, k, v; runs the T steps again) instead of the forward metric")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures ONE GPU (heads are independent problems: more GPUs would each take "
                 "a share of E*H with no communication) - run with --gpus 1")
    if args.record_traffic:
        record_traffic(args)
        return

    import torch

    from ma import _hip_lib as L
    from ma import ma_hip
    from ma.ma_hip import monarch_attention_hip
    from oracle.ma_oracle import forward_bytes, forward_flops, monarch_attention_oracle

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    lib = L.load()   # fails loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
    stream = torch.cuda.current_stream(dev)
    sp = stream.cuda_stream
    F = torch.nn.functional

    # The benchmark runs alone on its GPU and says so to the library (the fused kernel, whose
    # workgroups wait for each other, is only chosen for such callers): in the parameter blocks it
    # fills itself and, for the module-level leg, through the host wrapper's switch.
    EXCL = 0 if args.shared_device else L.MA_FLAG_DEVICE_EXCLUSIVE
    READY = L.MA_FLAG_SYNC_READY | EXCL
    ma_hip.DEVICE_EXCLUSIVE = not args.shared_device

    def make_params(*a, **kw):
        p = ma_hip.make_params(*a, **kw)
        p.flags = EXCL
        return p

    def checked(status):
        if status:
            L.check(status, "launch")

    def event_avg(fn, n):
        """Average duration (ms) of n back-to-back calls of fn between two events on the launch stream."""
        for i in range(3):
            fn(i)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(stream)
        for i in range(n):
            fn(i)
        b.record(stream)
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n

    def batch_stats(fn, steps):
        """median / min / mean ms per call over batches of 20 back-to-back calls."""
        per = 20
        nb = max(5, steps // per)
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(nb + 1)]
        evs[0].record(stream)
        for b in range(nb):
            for i in range(per):
                fn(b * per + i)
            evs[b + 1].record(stream)
        torch.cuda.synchronize()
        ts = [evs[b].elapsed_time(evs[b + 1]) / per for b in range(nb)]
        return {"median_ms": round(statistics.median(ts), 5), "min_ms": round(min(ts), 5), "mean_ms": round(statistics.fmean(ts), 5),
                "batches": nb, "calls_per_batch": per}

    # ------------------------------------------------------------------ the reference's sweep protocol
    if args.sweep_n or args.sweep_e:
        rows = []
        if args.sweep_n:
            # the reference's sweep ends at 2^14; 2^15 and 2^16 (blocks of 181 and 256 rows) are added here
            shapes = [(1, 12, 2 ** k, 64, int((2 ** k) ** 0.5)) for k in range(10, 17)]
            name = "sweep_n: fp16 E1 H12 D64, block floor(sqrt(N)), T=1 (perfbench/bench.py:87-127, extended to N = 2^16)"
        else:
            shapes = [(2 ** k, 12, 256, 64, 16) for k in range(3, 14)]
            name = "sweep_e: fp16 N256 H12 D64 block 16, T=1 (perfbench/bench.py:42-85)"
        for (E, H, N, D, B) in shapes:
            gen = torch.Generator().manual_seed(0)
            set_bytes = 4 * E * H * N * D * 2
            nbuf = max(2, min(16, -(-640 * 2 ** 20 // set_bytes)))
            base = [torch.randn(min(E, 64), H, N, D, generator=gen).to(torch.float16) for _ in range(3)]
            sets = []
            for i in range(nbuf):
                q, k, v = (t.to(dev).roll(i, dims=2).repeat(-(-E // t.shape[0]), 1, 1, 1)[:E].contiguous() for t in base)
                sets.append((q, k, v, torch.empty_like(q)))
            ps = [make_params(q, k, v, None, o, 1, B, False, "auto") for (q, k, v, o) in sets]
            nbytes = lib.ma_fwd_workspace_bytes(ps[0])
            ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
            for p in ps:
                p.workspace, p.workspace_bytes, p.flags = ws.data_ptr(), nbytes, READY
            variant = L.VARIANT_NAMES[lib.ma_fwd_select_variant(ps[0])]
            n = 100 if set_bytes < (1 << 30) else 20
            ma = batch_stats(lambda i: checked(lib.ma_fwd(ps[i % nbuf], sp)), n)
            sd = batch_stats(lambda i: F.scaled_dot_product_attention(*sets[i % nbuf][:3]), max(n // 2, 20))
            rows.append({"E": E, "H": H, "N": N, "D": D, "block": B, "variant": variant, "monarch": ma, "sdpa": sd,
                         "speedup_vs_sdpa": round(sd["median_ms"] / ma["median_ms"], 2),
                         "monarch_tflops": round(forward_flops(E, H, N, D, D, B, 1) / (ma["median_ms"] * 1e-3) / 1e12, 2),
                         "fwd_hbm_frac": round(forward_bytes(E, H, N, D, D, 2) / (ma["median_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)})
            del sets, ps, ws
            torch.cuda.empty_cache()
        faster = [r for r in rows if r["speedup_vs_sdpa"] > 1.0]
        print(json.dumps({"metric": "MonarchAttn fwd vs dense SDPA (reference sweep protocol)", "sweep": name, "unit": "ms",
                          "n_gpus": 1, "dtype": "f16", "data": "synthetic", "higher_is_better": False,
                          "first_faster_than_sdpa": ({"E": faster[0]["E"], "N": faster[0]["N"]} if faster else None),
                          "rows": rows}))
        return

    # ------------------------------------------------------------------ every variant over a grid of shapes
    if args.sweep_variants:
        T_, D = args.T or 2, args.head_dim
        # without the statement that the benchmark owns the device AUTO may not choose the team kernel: it is
        # then judged against the variants it may choose
        names = ("staged", "chained", "resident") if args.shared_device else ("staged", "chained", "fused", "resident")
        sdt = DT[args.sweep_dtype]
        selt = torch.empty((), dtype=sdt).element_size()
        rows, logsum, worst = [], 0.0, None
        if args.sweep_grid == "pow2":
            grid = [(h, N, B) for h in (1, 2, 4, 6, 8, 12, 16, 32, 64, 128, 192, 384) for N in (256, 512, 1024, 2048, 4096, 8192)
                    for B in (16, 32, 64, 128)]
        elif args.sweep_grid == "ragged":     # lengths of the reference's models: ViT 197, BART / RoBERTa prefixes, GPS graphs
            grid = [(h, N, B) for h in (2, 8, 12, 16, 48, 96, 192, 768) for (N, B) in ((197, 14), (197, 16), (500, 24), (1000, 32), (1000, 48),
                                                                                  (3000, 55), (3000, 64), (5000, 71), (5000, 128), (7600, 88), (7600, 128))]
        elif args.sweep_grid == "mid":        # heads of 256 .. 1000 tokens: the forms of the resident kernel against the rest
            grid = [(h, N, B) for h in (4, 16, 32, 64, 96, 128, 192, 256, 384, 512, 768)
                    for (N, B) in ((256, 16), (256, 32), (288, 16), (320, 32), (384, 16), (384, 24), (384, 32), (400, 25), (448, 32), (448, 64),
                                   (500, 24), (512, 16), (512, 32), (512, 64), (540, 36), (768, 32), (1000, 32))]
        elif args.sweep_grid == "short":      # hundreds to thousands of heads of at most 256 tokens (windows, patches): the narrow-workgroup forms
            grid = [(h, N, B) for h in (64, 128, 256, 384, 512, 768, 1024, 1536, 3072)
                    for (N, B) in ((49, 7), (64, 16), (96, 16), (128, 16), (128, 32), (160, 32), (197, 16), (224, 32), (256, 16))]
        elif args.sweep_grid == "fewheads":   # 8, 16, 24 heads of thousands of tokens: where the team kernel competes
            grid = [(h, N, B) for h in (8, 16, 24) for N in (2048, 4096, 5000, 6144, 8000, 8192) for B in (32, 64, 128)]
        else:   # blocks and / or block counts of 65 .. 96 rows (and two 128-row shapes with ragged block counts)
            grid = [(h, N, B) for h in (4, 8, 12, 16, 24, 32, 64, 192)
                    for (N, B) in ((8192, 96), (6000, 64), (4096, 48), (2048, 24), (1000, 80), (512, 96), (9000, 96), (5500, 80),
                                   (7000, 128), (12000, 128), (768, 96))]
        for (heads, N, B) in grid:
            M = -(-N // B)
            set_bytes = 4 * heads * N * D * selt
            if M > 128 or M < 2 or set_bytes > (1.2e9 if args.sweep_grid == "pow2" else 0.6e9):
                continue
            E, H = (heads // 4, 4) if heads % 4 == 0 else (1, heads)
            gen = torch.Generator().manual_seed(0)
            nbuf = max(2, min(8, -(-400 * 2 ** 20 // set_bytes)))
            base = [torch.randn(E, H, N, D, generator=gen).to(sdt) for _ in range(3)]
            sets = []
            for i in range(nbuf):
                q, k, v = (t.to(dev).roll(i, dims=2).contiguous() for t in base)
                sets.append((q, k, v, torch.empty_like(q)))
            mask = None
            if args.sweep_mask:   # a tokenizer-style int64 mask: the tail of every sequence masked out, at most 10 % of it
                keep = N - (torch.arange(E) * 7 % max(N // 10, 1))
                mask = (torch.arange(N)[None, :] < keep[:, None]).to(torch.int64).to(dev)
            row = {"heads": heads, "N": N, "block": B}
            for variant in ("auto",) + names:
                ps = [make_params(q, k, v, mask, o, T_, B, args.sweep_pre_pad, variant) for (q, k, v, o) in sets]
                sel = lib.ma_fwd_select_variant(ps[0])
                if variant == "auto":
                    row["auto"] = L.VARIANT_NAMES[sel]
                    continue
                if sel < 0:
                    continue
                nbytes = lib.ma_fwd_workspace_bytes(ps[0])
                ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
                for p in ps:
                    p.workspace, p.workspace_bytes, p.flags = ws.data_ptr(), nbytes, READY
                if any(lib.ma_fwd(ps[i % nbuf], sp) for i in range(4)):
                    continue   # e.g. a team grid that does not fit the device
                row[variant] = round(batch_stats(lambda i: checked(lib.ma_fwd(ps[i % nbuf], sp)), 100)["median_ms"] * 1e3, 2)
                del ws
            if row["auto"] not in row:   # AUTO went to a variant outside the list (the FMA kernels): nothing to judge it against
                continue
            best = min(names, key=lambda v: row.get(v, float("inf")))
            row["best"] = best
            row["auto_over_best"] = round(row[row["auto"]] / row[best], 3)
            logsum += math.log(row["auto_over_best"])
            if worst is None or row["auto_over_best"] > worst["auto_over_best"]:
                worst = row
            rows.append(row)
            del sets
            torch.cuda.empty_cache()
        print(json.dumps({"metric": "AUTO's choice against the fastest variant", "unit": "us (median)", "n_gpus": 1, "dtype": args.sweep_dtype,
                          "data": "synthetic", "T": T_, "D": D, "grid": args.sweep_grid, "points": len(rows),
                          "mask": bool(args.sweep_mask), "pre_pad": bool(args.sweep_pre_pad), "device_exclusive": not args.shared_device,
                          "geomean_auto_over_best": round(math.exp(logsum / max(len(rows), 1)), 4), "worst": worst, "rows": rows}))
        return

    E, H, N, D, B, T, dt, scale = CONFIGS[args.config]
    if args.T is not None:
        T = args.T
    dtype = DT[dt]
    elt = torch.empty((), dtype=dtype).element_size()

    # ---- synthetic inputs: torch.manual_seed(0), q, k, v = randn on the CPU in fp32, in that order
    gen = torch.Generator().manual_seed(0)
    base = [(scale * torch.randn(E, H, N, D, generator=gen)).to(dtype) for _ in range(3)]
    set_bytes = 4 * E * H * N * D * elt
    nbuf = max(2, min(64, -(-640 * 2**20 // set_bytes)))
    sets = []
    for i in range(nbuf):
        q, k, v = (t.to(dev).roll(i, dims=2).contiguous() for t in base)   # distinct addresses and contents
        sets.append((q, k, v, torch.empty(E, H, N, D, dtype=dtype, device=dev)))

    def prepared(T_, variant, rotate=None):
        """One ma_fwd_params per buffer set.  All sets share ONE zero-initialised workspace, as the
        calls of a model do (the host wrapper keeps one per device and stream), so the state arrays
        can stay in the 256 MB Infinity Cache between calls; with `rotate` every set has a workspace of
        its own (as long as they total at most 2 GiB) and the state rotates through memory like the inputs."""
        ps = [make_params(q, k, v, None, o, T_, B, False, variant) for (q, k, v, o) in sets]
        nbytes = lib.ma_fwd_workspace_bytes(ps[0])
        rotate = args.rotate_workspaces if rotate is None else rotate
        nws = max(1, min(nbuf, (2 << 30) // max(nbytes, 1))) if rotate else 1
        ws = [torch.zeros(nbytes, dtype=torch.uint8, device=dev) for _ in range(nws)]
        for i, p in enumerate(ps):
            p.workspace, p.workspace_bytes, p.flags = ws[i % nws].data_ptr(), nbytes, READY
        return ps, ws

    def run_steps(ps, n):
        fwd = lib.ma_fwd
        for i in range(n):
            st = fwd(ps[i % nbuf], sp)
            if st:
                L.check(st, "ma_fwd")

    def time_forward(T_, variant, steps, warmup, rotate=None):
        ps, ws = prepared(T_, variant, rotate)
        run_steps(ps, max(warmup, nbuf))
        # the timed region: exactly `steps` forward calls between two synchronisations, nothing else queued
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_steps(ps, steps)
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        # the same steps once more between two events on the launch stream (device-side time per step)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        run_steps(ps, steps)
        e1.record(stream)
        torch.cuda.synchronize()
        return wall_ms, e0.elapsed_time(e1) / steps, ps, ws

    if args.matrix:
        from ma.ma_hip import monarch_matrix_hip
        q, k, _, _ = sets[0]
        variant = args.variant if args.variant in ("auto", "generic", "staged") else "auto"
        for _ in range(3):
            monarch_matrix_hip(q, k, None, T, B, False, variant=variant)
        torch.cuda.synchronize()
        steps = max(args.steps // 20, 5)
        t0 = time.perf_counter()
        for _ in range(steps):
            monarch_matrix_hip(q, k, None, T, B, False, variant=variant)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        out_bytes = 4 * E * H * N * N
        print(json.dumps({"metric": "ma_matrix_ms", "value": round(ms, 4), "unit": "ms", "n_gpus": 1, "steps": steps,
                          "higher_is_better": False, "dtype": dt, "data": "synthetic",
                          "config": {"workload": f"{args.config}: E{E} H{H} N{N} D{D} block {B} T={T}", "variant": variant},
                          "output_bytes": out_bytes, "output_GBps": round(out_bytes / ms / 1e6, 1)}))
        return

    if args.backward:
        from ma.ma_hip import monarch_attention_hip_backward
        q, k, v, _ = sets[0]
        w = torch.randn(E, H, N, D, generator=gen).to(dtype).to(dev)
        variant = args.variant if args.variant in ("auto", "generic", "staged") else "auto"
        for _ in range(max(args.warmup // 10, 2)):
            monarch_attention_hip_backward(q, k, v, None, w, T, B, False, variant=variant)
        torch.cuda.synchronize()
        steps = max(args.steps // 10, 5)
        t0 = time.perf_counter()
        for _ in range(steps):
            monarch_attention_hip_backward(q, k, v, None, w, T, B, False, variant=variant)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3 / steps
        print(json.dumps({"metric": "ma_bwd_ms", "value": round(ms, 4), "unit": "ms", "n_gpus": 1, "steps": steps,
                          "higher_is_better": False, "dtype": dt, "data": "synthetic",
                          "config": {"workload": f"{args.config}: E{E} H{H} N{N} D{D} block {B} T={T}", "variant": variant}}))
        return

    M = -(-N // B)
    Np = M * B
    cbytes = forward_bytes(E, H, N, D, D, elt)
    mfma_peak = MFMA_PEAK_TFLOPS_F32 if dt == "f32" else MFMA_PEAK_TFLOPS

    def resolve(T_, variant):
        return L.VARIANT_NAMES[lib.ma_fwd_select_variant(make_params(*sets[0][:3], None, sets[0][3], T_, B, False, variant))]

    def roofline_of(T_, variant, ps, n):
        """Roofline entry of one forward with T_ steps: compulsory bytes over the summed average
        durations of the kernels it launches (events on the launch stream, back-to-back launches)."""
        res = resolve(T_, variant)
        stages = {}
        if res in ONE_LAUNCH:
            kernels = {lib.ma_fwd_kernel_name(ps[0]).decode(): (event_avg(lambda i: checked(lib.ma_fwd(ps[i % nbuf], sp)), n), 1)}
        else:
            # per-stage kernels on the state a full forward left in the workspace; (average ms, launches per forward)
            kernels = {"r_step(with V)": (event_avg(lambda i: checked(lib.ma_r_step(ps[i % nbuf], int(T_ == 1), 1, sp)), n), 1),
                       "z_step": (event_avg(lambda i: checked(lib.ma_z_step(ps[i % nbuf], sp)), n), 1)}
            stage_bytes = {"r_step(with V)": E * H * ((2 * N * D + N * D) * elt + 2 * Np * D * elt + 4 * Np),
                           "z_step": E * H * (N * D * elt + 2 * Np * D * elt + 4 * Np + N * D * elt)}
            if T_ > 1:
                kernels["l_step"] = (event_avg(lambda i: checked(lib.ma_l_step(ps[i % nbuf], sp)), n), T_ - 1)
                kernels["r_step"] = (event_avg(lambda i: checked(lib.ma_r_step(ps[i % nbuf], 0, 0, sp)), n), T_ - 1)
                stage_bytes["l_step"] = E * H * (N * D * elt + Np * D * elt + 4 * Np + Np * D * elt + 4 * Np)
                stage_bytes["r_step"] = E * H * (2 * N * D * elt + Np * D * elt + 4 * Np + 4 * Np)
            # secondary figure per stage: bytes INCLUDING the state it reads and writes over its own duration
            stages = {k: {"avg_launch_us": round(v[0] * 1e3, 2), "launches_per_forward": v[1],
                          "bytes_incl_intermediates": stage_bytes[k],
                          "stage_copy_frac": round(stage_bytes[k] / (v[0] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)} for k, v in kernels.items()}
        fwd_ms = sum(ms_ * cnt for ms_, cnt in kernels.values())
        dom = max(kernels, key=lambda k: kernels[k][0] * kernels[k][1])
        achieved = cbytes / (fwd_ms * 1e-3) / 1e9
        r = {"bound": "hbm", "T": T_, "variant": res, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
             "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": recorded_traffic(args.config, T_, variant),
             "algorithmic_bytes_per_forward": cbytes, "kernel_time_per_forward_us": round(fwd_ms * 1e3, 2),
             "kernel": dom, "kernel_share": round(kernels[dom][0] * kernels[dom][1] / fwd_ms, 3),
             "kernels_us": {k: round(v[0] * 1e3, 2) for k, v in kernels.items()},
             "mfma_frac": round(forward_flops(E, H, N, D, D, B, T_) / (fwd_ms * 1e-3) / 1e12 / mfma_peak, 5)}
        if stages:
            r["stages"] = stages
        return r

    resolved = resolve(T, args.variant)
    flops = forward_flops(E, H, N, D, D, B, T)

    # ---- the timed region: exactly K steps between two synchronisations
    wall_ms, ev_ms, ps, ws = time_forward(T, args.variant, args.steps, args.warmup)
    ms = wall_ms
    timing = batch_stats(lambda i: checked(lib.ma_fwd(ps[i % nbuf], sp)), max(args.steps, 100))
    roofline = roofline_of(T, args.variant, ps, min(max(args.steps, 100), 200))

    out = {
        "metric": "MonarchAttn fwd TFLOP/s (fp16 B1 H16 N4096 d64, b=64)" if args.config == "cM" else f"MonarchAttn fwd TFLOP/s ({args.config})",
        "value": round(flops / (ms * 1e-3) / 1e12, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dt, "data": "synthetic",
        "config": {"workload": f"{args.config}: {dt} E{E} H{H} N{N} D{D} block{B} T{T} post-pad no-mask", "variant": resolved,
                   "flop_per_fwd": flops, "compulsory_bytes_per_fwd": cbytes, "rotating_input_sets": nbuf, "rotating_workspaces": len(ws),
                   "device_exclusive": not args.shared_device},
        "stream_ms_per_step": round(ev_ms, 5),
        "ms_per_step_stats": timing,
        "fwd_hbm_frac": round(cbytes / (ev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "fwd_mfma_frac": round(flops / (ev_ms * 1e-3) / 1e12 / mfma_peak, 5),
        "roofline": roofline,
    }
    del ps, ws

    # ---- the same forward through the nn.Module-level host wrapper (allocates its output per call)
    q0, k0, v0, _ = sets[0]
    for _ in range(5):
        monarch_attention_hip(q0, k0, v0, None, T, B, False, variant=args.variant)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    nmod = min(args.steps, 200)
    for i in range(nmod):
        q, k, v, _ = sets[i % nbuf]
        monarch_attention_hip(q, k, v, None, T, B, False, variant=args.variant)
    torch.cuda.synchronize()
    out["module_ms_per_step"] = round((time.perf_counter() - t0) * 1e3 / nmod, 5)

    # ---- T = 1, 2, 3 with the selected variant: one roofline entry each; and every variant (same protocol, fewer steps)
    if not args.no_sweep:
        # the same K steps with a workspace per input set: what the Infinity Cache contributes to the state exchange
        _, rot_ms, ps, ws = time_forward(T, args.variant, max(args.steps, 100), max(args.warmup, 10), rotate=True)
        out["stream_ms_per_step_rotating_workspaces"] = round(rot_ms, 5)
        out["config"]["rotating_workspaces_in_that_run"] = len(ws)
        del ps, ws
        by_T = []
        for T_ in (1, 2, 3):
            ps_, ws_ = prepared(T_, args.variant)
            run_steps(ps_, max(10, nbuf))   # every workspace holds the state of a full forward
            by_T.append(roofline_of(T_, args.variant, ps_, 100))
            del ps_, ws_
        out["roofline_by_T"] = by_T
        sweep = {}
        for T_ in (1, 2, 3):
            for variant in ("staged", "fused", "chained", "resident"):
                try:
                    _, ems, _, _ = time_forward(T_, variant, max(50, args.steps // 4), 10)
                except (NotImplementedError, ValueError):
                    continue
                f_ = forward_flops(E, H, N, D, D, B, T_)
                sweep[f"T{T_}_{variant}"] = {"ms": round(ems, 5), "tflops": round(f_ / (ems * 1e-3) / 1e12, 3),
                                            "hbm_frac": round(cbytes / (ems * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
        out["sweep"] = sweep

    # ---- dense softmax attention on the same GPU (PyTorch's own SDPA backend), same harness
    if not args.no_sdpa and dt != "f32":
        for _ in range(3):
            F.scaled_dot_product_attention(q0, k0, v0)
        torch.cuda.synchronize()
        ns = max(10, min(100, args.steps // 4))
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(ns):
            q, k, v, _ = sets[i % nbuf]
            F.scaled_dot_product_attention(q, k, v)
        e1.record(stream)
        torch.cuda.synchronize()
        sd = e0.elapsed_time(e1) / ns
        out["sdpa_dense"] = {"ms": round(sd, 5), "speedup_of_monarch": round(sd / ev_ms, 2),
                             "dense_tflops": round(4 * N * N * D * E * H / (sd * 1e-3) / 1e12, 2)}

    # ---- CPU baseline: the oracle (port of ma_torch.py) on this host's cores, bounded sample
    if not args.no_cpu:
        qc, kc, vc = (t.float() for t in base)            # fp32 is the fair CPU dtype (16-bit GEMMs are slow paths)
        heads = min(H, 16)
        if args.config == "c5":
            heads = 4
        qc, kc, vc = qc[:1, :heads], kc[:1, :heads], vc[:1, :heads]
        monarch_attention_oracle(qc, kc, vc, None, T, B, False)   # warm-up
        runs, t_cpu = 0, []
        t_start = time.perf_counter()
        while runs < 3 or (time.perf_counter() - t_start < 10.0 and runs < 50):
            t0 = time.perf_counter()
            monarch_attention_oracle(qc, kc, vc, None, T, B, False)
            t_cpu.append(time.perf_counter() - t0)
            runs += 1
        t_med = sorted(t_cpu)[len(t_cpu) // 2]
        f_cpu = forward_flops(1, heads, N, D, D, B, T)
        out["cpu_baseline"] = {"value": round(f_cpu / t_med / 1e12, 5), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
                               "kind": "port", "ms_per_fwd_equiv": round(t_med * 1e3 * (E * H) / heads, 3),
                               "sample": f"oracle (fp32 tensors, torch CPU ops) on E1 x H{heads} of the workload, median of {runs} runs, "
                                         f"host cpu_count={os.cpu_count()}"}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
