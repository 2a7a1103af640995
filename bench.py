#!/usr/bin/env python3
"""Benchmark of the MonarchAttention forward pass on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config cM] [--T 1]
                    [--variant auto|generic|staged|fused|resident|chained] [--no-cpu] [--no-sdpa] [--no-sweep]

A step is ONE forward call of the hot path (monarch_attention, all T steps)
through the C ABI on synthetic inputs that are already resident in HBM.  The
default workload is the configuration the headline metric is quoted on: fp16,
E=1, H=16, N=4096, D=64, block B=64 (=sqrt(N)), post-pad, no mask, with T=1 as in
the reference's own micro-benchmark protocol (perfbench/bench.py:427-431); the
sweep over T = 1, 2, 3 is reported next to it.  Inputs rotate over enough
distinct (q, k, v, out) sets to exceed the 256 MB Infinity Cache, so every step
reads its operands from HBM.

Prints ONE JSON line.  `value` is the forward throughput in TFLOP/s (matmul
FLOPs on padded sizes, the reference's bmm convention,
experiments/vit/evaluation.py:50-59); `roofline` prices the dominant kernel's
algorithmic bytes against the 8 TB/s HBM peak using that kernel's average
duration measured with HIP events on the launch stream; `cpu_baseline` is the
CPU oracle (a port of the reference's ma_torch.py) timed on this host.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "monarch-attention_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

CONFIGS = {  # name: (E, H, N, D, B, T, dtype, scale)  - BASELINE.json configs + the metric configuration
    "cM": (1, 16, 4096, 64, 64, 1, "f16", 1.0),
    "c1": (1, 1, 256, 64, 16, 1, "f32", 1.0),
    "c2": (64, 12, 197, 64, 16, 2, "f16", 0.125),
    "c2b": (64, 12, 256, 64, 16, 2, "f16", 0.125),
    "c3": (16, 12, 512, 64, 32, 2, "bf16", 1.0),
    "c4": (8, 16, 1024, 72, 32, 3, "f16", 1.0),
    "c5": (1, 16, 16384, 64, 128, 3, "f16", 1.0),
    # model shapes beyond the BASELINE configs (fp32 goes through the fp32 matrix-core stage kernels)
    "gps": (1, 2, 7600, 48, 128, 2, "f32", 1.0),
    "c3f32": (16, 12, 512, 64, 32, 2, "f32", 1.0),
    "bart": (2, 16, 8192, 64, 64, 2, "bf16", 1.0),
}
HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E peak
MFMA_PEAK_TFLOPS = 2500.0      # dense fp16 / bf16
MFMA_PEAK_TFLOPS_F32 = 157.3   # dense fp32

# HBM-side bytes per launch of the dominant kernels on the metric workload, from rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE runs of this script, each scaled by what the same counter reads for a plain
# 256 MiB device copy (FETCH_SIZE x 2.00, WRITE_SIZE x 1.00); see profiles/traffic_cM_T1.md.
MEASURED_TRAFFIC_BYTES = {
    ("cM", 1, "r_step(with V)"): 44_188_000,
    ("cM", 1, "z_step"): 33_935_000,
    ("cM", 1, "fused_fwd_mfma"): 71_980_000,
    ("cM", 1, "chain_fwd_mfma"): 70_300_000,
    ("c3", 2, "chain_fwd_mfma"): 175_100_000,
    ("c2", 2, "resident_fwd_mfma"): 102_330_000,
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=400)
    ap.add_argument("--warmup", type=int, default=40)
    ap.add_argument("--config", default="cM", choices=sorted(CONFIGS))
    ap.add_argument("--T", type=int, default=None, help="override the number of alternating steps")
    ap.add_argument("--variant", default="auto", choices=["auto", "generic", "staged", "fused", "resident", "chained"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-sdpa", action="store_true", help="skip the dense SDPA comparison")
    ap.add_argument("--no-sweep", action="store_true", help="skip the T = 1, 2, 3 sweep")
    ap.add_argument("--matrix", action="store_true",
                    help="time ma_matrix (the dense (E,H,N,N) attention matrix of get_matrix) instead of the forward metric")
    ap.add_argument("--backward", action="store_true",
                    help="time ma_bwd (gradients of q, k, v; runs the T steps again) instead of the forward metric")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures ONE GPU (heads are independent problems: more GPUs would each take "
                 "a share of E*H with no communication) - run with --gpus 1")

    import torch

    from ma import _hip_lib as L
    from ma.ma_hip import make_params, monarch_attention_hip
    from oracle.ma_oracle import forward_bytes, forward_flops, monarch_attention_oracle

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    lib = L.load()   # fails loudly if the HIP library is missing
    dev = torch.device("cuda:0")
    DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
    E, H, N, D, B, T, dt, scale = CONFIGS[args.config]
    if args.T is not None:
        T = args.T
    dtype = DT[dt]
    elt = torch.empty((), dtype=dtype).element_size()
    stream = torch.cuda.current_stream(dev)

    # ---- synthetic inputs: torch.manual_seed(0), q, k, v = randn on the CPU in fp32, in that order
    gen = torch.Generator().manual_seed(0)
    base = [(scale * torch.randn(E, H, N, D, generator=gen)).to(dtype) for _ in range(3)]
    set_bytes = 4 * E * H * N * D * elt
    nbuf = max(2, min(64, -(-640 * 2**20 // set_bytes)))
    sets = []
    for i in range(nbuf):
        q, k, v = (t.to(dev).roll(i, dims=2).contiguous() for t in base)   # distinct addresses and contents
        sets.append((q, k, v, torch.empty(E, H, N, D, dtype=dtype, device=dev)))

    def prepared(T_, variant):
        """One ma_fwd_params per buffer set, all on one zero-initialised workspace."""
        ps = [make_params(q, k, v, None, o, T_, B, False, variant) for (q, k, v, o) in sets]
        nbytes = lib.ma_fwd_workspace_bytes(ps[0])
        ws = torch.zeros(nbytes, dtype=torch.uint8, device=dev)
        for p in ps:
            p.workspace, p.workspace_bytes, p.flags = ws.data_ptr(), nbytes, L.MA_FLAG_SYNC_READY
        return ps, ws

    def run_steps(ps, n):
        sp = stream.cuda_stream
        fwd = lib.ma_fwd
        for i in range(n):
            st = fwd(ps[i % nbuf], sp)
            if st:
                L.check(st, "ma_fwd")

    def time_forward(T_, variant, steps, warmup):
        ps, ws = prepared(T_, variant)
        run_steps(ps, warmup)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(stream)
        run_steps(ps, steps)
        e1.record(stream)
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
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

    resolved = L.VARIANT_NAMES[lib.ma_fwd_select_variant(make_params(*sets[0][:3], None, sets[0][3], T, B, False, args.variant))]
    flops = forward_flops(E, H, N, D, D, B, T)
    cbytes = forward_bytes(E, H, N, D, D, elt)

    # ---- the timed region: exactly K steps between two synchronisations
    wall_ms, ev_ms, ps, ws = time_forward(T, args.variant, args.steps, args.warmup)
    ms = wall_ms

    # ---- dominant kernel: average launch duration with HIP events on the launch stream
    def event_avg(fn, n):
        """Average duration of n back-to-back launches of one kernel between two events."""
        for i in range(3):
            fn(i)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(stream)
        for i in range(n):
            fn(i)
        b.record(stream)
        torch.cuda.synchronize()
        return a.elapsed_time(b) / n

    sp = stream.cuda_stream
    M = -(-N // B)
    Np = M * B
    kernels = {}
    def checked(status):
        if status:
            L.check(status, "stage launch")

    if resolved in ("fused", "resident", "chained"):   # the whole forward is one kernel
        kname = {"fused": "fused_fwd_mfma", "resident": "resident_fwd_mfma", "chained": "chain_fwd_mfma"}[resolved]
        kernels[kname] = (event_avg(lambda i: checked(lib.ma_fwd(ps[i % nbuf], sp)), min(args.steps, 200)), cbytes)
    else:
        # per-stage kernels on the state a full forward left in the workspace
        n = min(args.steps, 200)
        rv_bytes = E * H * ((2 * N * D + N * D) * elt + 2 * Np * D * elt + 4 * Np)          # Q,K,V -> aL,Y,cL
        kernels["r_step(with V)"] = (event_avg(lambda i: checked(lib.ma_r_step(ps[i % nbuf], int(T == 1), 1, sp)), n), rv_bytes)
        z_bytes = E * H * (N * D * elt + 2 * Np * D * elt + 4 * Np + N * D * elt)            # Q,aL,Y,cL -> out
        kernels["z_step"] = (event_avg(lambda i: checked(lib.ma_z_step(ps[i % nbuf], sp)), n), z_bytes)
        if T > 1:
            l_bytes = E * H * (N * D * elt + Np * D * elt + 4 * Np + Np * D * elt + 4 * Np)  # Q,aL,cL -> aR,cR
            kernels["l_step"] = (event_avg(lambda i: checked(lib.ma_l_step(ps[i % nbuf], sp)), n), l_bytes)
            r_bytes = E * H * (2 * N * D * elt + Np * D * elt + 4 * Np + 4 * Np)              # aR,cR,K -> aL,cL
            kernels["r_step"] = (event_avg(lambda i: checked(lib.ma_r_step(ps[i % nbuf], 0, 0, sp)), n), r_bytes)
    dom = max(kernels, key=lambda kname: kernels[kname][0])
    dom_ms, dom_bytes = kernels[dom]
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": dom, "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": MEASURED_TRAFFIC_BYTES.get((args.config, T, dom)),
                "algorithmic_bytes_per_launch": dom_bytes, "avg_launch_us": round(dom_ms * 1e3, 2),
                "kernels_us": {kname: round(v[0] * 1e3, 2) for kname, v in kernels.items()}}

    out = {
        "metric": "MonarchAttn fwd TFLOP/s (fp16 B1 H16 N4096 d64, b=64)" if args.config == "cM" else f"MonarchAttn fwd TFLOP/s ({args.config})",
        "value": round(flops / (ms * 1e-3) / 1e12, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 5), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": dt, "data": "synthetic",
        "config": {"workload": f"{args.config}: {dt} E{E} H{H} N{N} D{D} block{B} T{T} post-pad no-mask", "variant": resolved,
                   "flop_per_fwd": flops, "compulsory_bytes_per_fwd": cbytes, "rotating_input_sets": nbuf},
        "stream_ms_per_step": round(ev_ms, 5),
        "fwd_hbm_frac": round(cbytes / (ev_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "fwd_mfma_frac": round(flops / (ev_ms * 1e-3) / 1e12 / (MFMA_PEAK_TFLOPS_F32 if dt == "f32" else MFMA_PEAK_TFLOPS), 5),
        "roofline": roofline,
    }

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

    # ---- sweep over T and variants (same protocol, fewer steps)
    if not args.no_sweep:
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
        F = torch.nn.functional
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
