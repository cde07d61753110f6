#!/usr/bin/env python3
"""Benchmark of the recurrent hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C2] [--backend hip_fused]
    python bench.py --shape lstm:bfloat16:16:1024:1:768 --no-cpu      (any other shape: function:dtype:B:T:N:D)

A step is one forward + backward pass of ``flashrnn()`` over one batch of synthetic input that is
already resident in HBM.  Prints ONE JSON line: tokens/s (B*T per second) of the whole job, the
roofline figures of the dominant kernel (measured with HIP events on the launch stream inside the
timed region), the same workload on the alternating backend, and the CPU oracle timed on the host.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# name -> workload; seeds fixed per config.  C2 is the configuration the metric is quoted on.
WORKLOADS = {
    "C1": dict(function="lstm", dtype="float32", B=4, T=256, N=1, D=64, init="zeros", grad_on="all", bwd=False, seed=1001),
    "C2": dict(function="lstm", dtype="bfloat16", B=8, T=1024, N=3, D=256, init="randn", grad_on="all", bwd=True, seed=1002),
    "C3": dict(function="gru", dtype="bfloat16", B=16, T=2048, N=4, D=128, init="zeros", grad_on="all", bwd=True, seed=1003),
    "C4": dict(function="slstm", dtype="bfloat16", B=16, T=4096, N=4, D=192, init="zeros", grad_on="h", bwd=True, seed=1004,
               forget_bias_linspace=True),
    "C5": dict(function="elman", dtype="bfloat16", B=32, T=1024, N=1, D=1024, init="zeros", grad_on="all", bwd=True, seed=1005),
}
GATES_R = {"lstm": 4, "slstm": 4, "gru": 3, "elman": 1}
PEAK_TFLOPS = {"bfloat16": 2500.0, "float16": 2500.0, "float32": 157.3}  # MI355X dense MFMA, published
# roofline.traffic comes from the committed counter profiles of the same commands, never from a constant in this file:
# a profile holds one "traffic:" line per kernel template it measured (FETCH_SIZE and WRITE_SIZE in KiB per dispatch
# and the factors a plain 256 MiB copy gave in the same run; for the alternating backend per call, all step launches
# together).  Every profiles/*_counters*.txt is searched.  If the kernel that ran here is not a template that was
# profiled (another tiling, tile height or mode), traffic is null and the reason is given.
PROFILES = os.path.join(ROOT, "profiles")
CELL_NAMES = {"lstm": "LSTM", "slstm": "sLSTM", "gru": "GRU", "elman": "Elman"}


def kernel_template(w, kernel, recompute):
    """Name of the fused kernel instantiation this workload runs, as the profiles spell it."""
    from flashrnn_amd import fused_plan

    backward = kernel == "fused_bwd_kernel"
    waves, utw, kw, active = fused_plan(w["function"], w["dtype"], w["B"], w["N"], w["D"], backward)
    tiles = active // kw // w["N"]
    tr = next(t for t in (4, 8, 16) if (w["B"] + t - 1) // t == tiles)
    rc = ",RECOMPUTE" if (recompute and backward and w["function"] != "elman") else ""
    dt = {"bfloat16": "bf16", "float32": "f32", "float16": "f16"}[w["dtype"]]
    return f"{kernel}<{CELL_NAMES[w['function']]},{dt},D={w['D']},WAVES={waves},UTW={utw},KW={kw},TILE_ROWS={tr}{rc}>"


def profiled_traffic(w, kernel, recompute):
    """(bytes per launch or None, note)."""
    import glob

    if kernel in ("alt_forward_steps", "alt_backward_steps"):
        name = kernel  # (the benchmark's launch is the whole scan: every step kernel of one call)
        wanted = f"{w['function']}_{ {'bfloat16': 'bf16', 'float32': 'f32', 'float16': 'f16'}[w['dtype']] }_B{w['B']}_T{w['T']}_N{w['N']}_D{w['D']}".replace(" ", "")
    else:
        wanted = None
        try:
            name = kernel_template(w, kernel, recompute)
        except Exception as e:
            return None, f"no fused kernel template for this run ({e})"
    mode = "recomputed" if recompute else "stored"
    files = sorted(glob.glob(os.path.join(PROFILES, "*counters*.txt")))
    if not files:
        return None, "no counter profiles under profiles/"
    for path in files:
        if wanted is not None and wanted not in os.path.basename(path):
            continue  # (an aggregate of step kernels only means something for the workload it was measured on)
        for l in open(path):
            if not l.startswith("traffic:"):
                continue
            f = dict(x.split("=", 1) for x in l.split()[1:])
            if f["kernel"] == name and f["mode"] == mode:
                b = float(f["fetch_kib"]) * 1024 / float(f["fetch_factor"]) + float(f["write_kib"]) * 1024 / float(f["write_factor"])
                rel = os.path.relpath(path, ROOT)
                return b, (f"{rel}: FETCH_SIZE {f['fetch_kib']} KiB / {f['fetch_factor']} + WRITE_SIZE {f['write_kib']} KiB / "
                           f"{f['write_factor']} (factors of a plain 256 MiB copy in the same run)")
    return None, f"no committed profile has an entry for {name} (gate cache {mode}): not measured"


def describe(w):
    return (f"{w['function']} {w['dtype']} B{w['B']} T{w['T']} N{w['N']} D{w['D']} "
            f"{'fwd+bwd' if w['bwd'] else 'fwd'}")


def make_gpu_inputs(w, device):
    import torch
    from oracle import make_inputs

    kdt = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32}[w["dtype"]]
    rt = kdt if kdt != torch.float32 else None
    inp = make_inputs(w["function"], w["B"], w["T"], w["N"], w["D"], w["seed"], init=w["init"], round_to=rt,
                      grad_on=w["grad_on"], forget_bias_linspace=w.get("forget_bias_linspace", False))
    dev = {k: v.to(device=device, dtype=kdt) for k, v in inp.items()}
    return inp, dev


def run_gpu(w, backend, steps, warmup, device, recompute=False):
    """Returns (ms_per_step, {kernel name: (avg ms, launches per step)})."""
    import torch
    from flashrnn_amd import FlashRNNConfig, flashrnn, load_library

    lib = load_library()
    _, dev = make_gpu_inputs(w, device)
    leaves = [dev[k].requires_grad_(w["bwd"]) for k in ("Wx", "R", "b", "states")]
    dst = dev["dstates"]

    cfg = FlashRNNConfig(backend=backend, function=w["function"], dtype=w["dtype"], head_dim=w["D"], num_heads=w["N"],
                         batch_size=w["B"], recompute_gates=bool(recompute and backend == "hip_fused"))

    def step():
        out, _ = flashrnn(*leaves, config=cfg)
        if w["bwd"]:
            torch.autograd.grad(out, leaves, grad_outputs=dst)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    # profile entries that one step produces (it depends on the tiling: heads of one workgroup have no clearing launch)
    lib.frnn_profile_enable(1)
    step()
    torch.cuda.synchronize()
    entries_per_step = max(1, lib.frnn_profile_count())
    lib.frnn_profile_enable(0)
    # HIP events around every kernel launch, recorded on the launch stream inside the timed
    # region; the library keeps the most recent 64 launches, read after the region ends
    lib.frnn_profile_enable(1)
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    per_kernel = {}
    held = lib.frnn_profile_count()
    for i in range(held):
        per_kernel.setdefault(lib.frnn_profile_name(i).decode(), []).append(lib.frnn_profile_ms(i))
    lib.frnn_profile_enable(0)
    # (steps that the ring of launches holds: a fraction when a step has more entries than fit a whole number of times)
    calls = max(1.0, min(float(steps), held / entries_per_step))
    kern = {k: (sum(v) / len(v), max(1, round(len(v) / calls))) for k, v in per_kernel.items()}
    return (t1 - t0) * 1e3 / steps, kern


def run_with_linear(w, backend, steps, warmup, device):
    """The reference's "withlinear" benchmark variants (speed_experiments/kernel_speed_benchmark.py:387-407): the input
    projection Wx = Linear(x) in front of the recurrence, forward and backward through both.  The kernels read the
    [B, T, G, N, D] tensor that the Linear writes as it is (a view of its [B, T, G*N*D] output): no permuted copy lies
    between the two, which is the whole of the fusion that the reference measures.  Returns ms per step."""
    import torch
    from flashrnn_amd import FlashRNNConfig, flashrnn

    _, dev = make_gpu_inputs(w, device)
    B, T, N, D = w["B"], w["T"], w["N"], w["D"]
    Gw = dev["Wx"].shape[2]
    F = N * D
    g = torch.Generator(device="cpu").manual_seed(w["seed"] + 7)
    x = torch.randn((B, T, F), generator=g).to(device, dev["Wx"].dtype).requires_grad_(True)
    W = (torch.randn((Gw * N * D, F), generator=g) / F ** 0.5).to(device, dev["Wx"].dtype).requires_grad_(True)
    rest = [dev[k].requires_grad_(w["bwd"]) for k in ("R", "b", "states")]
    cfg = FlashRNNConfig(backend=backend, function=w["function"], dtype=w["dtype"], head_dim=D, num_heads=N, batch_size=B)

    def step():
        Wx = torch.nn.functional.linear(x, W).view(B, T, Gw, N, D)
        out, _ = flashrnn(Wx, *rest, config=cfg)
        if w["bwd"]:
            torch.autograd.grad(out, [x, W] + rest, grad_outputs=dev["dstates"])

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def run_cpu_baseline(w, budget_s=20.0):
    """The CPU oracle (a port of the reference's vanilla backend) on the host cores, fp32, on a bounded
    sample: the first T_cpu time steps of the workload, T_cpu chosen from a 32-step probe so that one
    pass takes about 8 s (the whole sequence if that is shorter: C1, C2)."""
    import torch
    from oracle import flashrnn_oracle, make_inputs

    torch.set_num_threads(os.cpu_count() or 1)
    rt = torch.bfloat16 if w["dtype"] == "bfloat16" else None
    T_full = w["T"]

    def make(T):
        wc = dict(w, T=T)
        inp = make_inputs(wc["function"], wc["B"], T, wc["N"], wc["D"], wc["seed"], init=wc["init"], round_to=rt,
                          grad_on=wc["grad_on"], forget_bias_linspace=wc.get("forget_bias_linspace", False))

        def one():
            leaves = [inp[k].clone().requires_grad_(w["bwd"]) for k in ("Wx", "R", "b", "states")]
            out, _ = flashrnn_oracle(*leaves, function=w["function"], slstm_per_element_first_step=True)
            if w["bwd"]:
                torch.autograd.grad(out, leaves, grad_outputs=inp["dstates"])
        return one

    probe_T = min(T_full, 32)
    probe = make(probe_T)
    probe()
    t0 = time.perf_counter()
    probe()
    per_step = (time.perf_counter() - t0) / probe_T
    T_cpu = max(probe_T, min(T_full, int(8.0 / max(per_step, 1e-6))))
    one = make(T_cpu)
    t0 = time.perf_counter()
    one()  # warm-up, also tells us how many repetitions fit the budget
    first = time.perf_counter() - t0
    reps = max(1, min(5, int(budget_s / max(first, 1e-3))))
    times = []
    for _ in range(reps):
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    sample = "full workload" if T_cpu == T_full else f"first {T_cpu} of {T_full} time steps"
    return dict(value=w["B"] * T_cpu / med, unit="tokens/s", cores=torch.get_num_threads(), kind="port",
                sample=f"{sample} ({describe(w)}), fp32 torch CPU, median of {reps} after 1 warm-up",
                ms=med * 1e3)


def run_sweep(device, steps, warmup):
    """The fused-path head-dim sweep of the fifth configuration (LSTM bf16 B16 T1024, N*D = 768; D = 512 has N = 1)
    on both backends, and the fifth configuration itself (Elman D = 1024 B32) on both."""
    rows = []
    for N, D in ((24, 32), (12, 64), (6, 128), (3, 256), (1, 512)):
        w = dict(function="lstm", dtype="bfloat16", B=16, T=1024, N=N, D=D, init="zeros", grad_on="all", bwd=True, seed=1006)
        r = {"workload": describe(w)}
        for backend in ("hip_fused", "hip"):
            ms, _ = run_gpu(w, backend, steps if backend == "hip_fused" else max(3, steps // 4), warmup, device)
            r[backend + "_ms"] = ms
        r["tokens_per_s_hip_fused"] = 16 * 1024 / (r["hip_fused_ms"] * 1e-3)
        r["speedup_of_hip_fused"] = r["hip_ms"] / r["hip_fused_ms"]
        rows.append(r)
    w5 = WORKLOADS["C5"]
    r = {"workload": describe(w5)}
    for backend in ("hip", "hip_fused"):
        ms, _ = run_gpu(w5, backend, max(3, steps // 2), warmup, device)
        r[backend + "_ms"] = ms
    r["note"] = "the configuration names the alternating backend (hip); the fused kernels also cover this head dim and are faster"
    rows.append(r)
    return rows


def run_steps(device, n_steps=256):
    """Single-step decoding (flashrnn_step with the fp32 carry): microseconds per step, eager and replayed from a
    HIP graph of 64 chained steps (the device-side cost of a dependent step), and the step kernel between two HIP
    events (which resolve ~6 us at best)."""
    import torch
    from flashrnn_amd import flashrnn_step, load_library, make_carry
    from oracle import make_inputs

    lib = load_library()
    out = []
    for function, N, D in (("lstm", 3, 256), ("lstm", 4, 192), ("lstm", 12, 64), ("gru", 4, 128), ("slstm", 4, 192)):
        for B in (1, 8):
            for backend in ("hip_fused", "hip"):
                inp = make_inputs(function, B, 1, N, D, 7, init="randn", round_to=torch.bfloat16)
                x = {k: v.to(device, torch.bfloat16).contiguous() for k, v in inp.items()}
                carry = make_carry(x["states"])
                kw = dict(function=function, backend=backend, dtype="bfloat16", carry=carry)
                s = x["states"]
                for _ in range(20):
                    s = flashrnn_step(x["Wx"], x["R"], x["b"], s, **kw)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(n_steps):
                    s = flashrnn_step(x["Wx"], x["R"], x["b"], s, **kw)
                torch.cuda.synchronize()
                eager = (time.perf_counter() - t0) / n_steps * 1e6
                lib.frnn_profile_enable(1)
                for _ in range(32):
                    s = flashrnn_step(x["Wx"], x["R"], x["b"], s, **kw)
                torch.cuda.synchronize()
                ks = [lib.frnn_profile_ms(i) * 1e3 for i in range(lib.frnn_profile_count())]
                lib.frnn_profile_enable(0)
                # one graph of 64 chained steps (each reads the states the one before wrote): its replay time / 64 is
                # the device-side cost of a dependent step, free of host time and of the event resolution
                CH = 64
                s_in = x["states"].clone()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    s_c = s_in
                    for _ in range(CH):
                        s_c = flashrnn_step(x["Wx"], x["R"], x["b"], s_c, **kw)
                    s_in.copy_(s_c)
                for _ in range(5):
                    g.replay()
                torch.cuda.synchronize()
                reps = max(1, n_steps // CH)
                t0 = time.perf_counter()
                for _ in range(reps):
                    g.replay()
                torch.cuda.synchronize()
                graph = (time.perf_counter() - t0) / (reps * CH) * 1e6
                out.append({"cell": f"{function} bf16 B{B} N{N} D{D}", "backend": backend, "eager_us_per_step": eager,
                            "graph_replay_us_per_step": graph, "kernel_event_us": sorted(ks)[len(ks) // 2]})
    return out


def run_decode(device, n_tokens=256):
    """The resident decode kernel (FlashRNNDecoder): microseconds per token, (a) one token per post, eager; (b) the
    same replayed from a HIP graph of 64 chained posts, each of which ends when it has collected its token: the
    device-side cost of a token whose input depends on the previous output; (c) 16 tokens per post, replayed: the
    rate at which the resident kernel serves tokens that are already there."""
    import torch
    from flashrnn_amd import FlashRNNDecoder
    from oracle import make_inputs

    out = []
    side = torch.cuda.Stream()
    for function, N, D in (("lstm", 3, 256), ("lstm", 4, 192), ("lstm", 12, 64), ("gru", 4, 128), ("slstm", 4, 192)):
        for B in (1, 8):
            inp = make_inputs(function, B, 16, N, D, 7, init="randn", round_to=torch.bfloat16)
            x = {k: v.to(device, torch.bfloat16).contiguous() for k, v in inp.items()}
            wx1, wx16 = x["Wx"][:, :1].contiguous(), x["Wx"].contiguous()
            S = x["states"].shape[0]
            o1 = torch.empty((S, B, 1, N, D), dtype=torch.bfloat16, device=device)
            o16 = torch.empty((S, B, 16, N, D), dtype=torch.bfloat16, device=device)
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):  # (graph capture needs a stream other than the default one)
                dec = FlashRNNDecoder(x["R"], x["b"], x["states"], function=function, slots=16, idle_polls=1 << 23)
                for _ in range(20):
                    dec.step(wx1, out=o1)
                side.synchronize()
                t0 = time.perf_counter()
                for _ in range(n_tokens):
                    dec.step(wx1, out=o1)
                side.synchronize()
                eager = (time.perf_counter() - t0) / n_tokens * 1e6

                graphs = []  # (kept until the session is closed: destroying a graph frees memory, which waits for the device)

                def replayed(wx, o, launches):
                    # (capture_begin / capture_end: the torch.cuda.graph context manager synchronises the device)
                    g = torch.cuda.CUDAGraph()
                    graphs.append(g)
                    g.capture_begin()
                    for _ in range(launches):
                        dec.step(wx, out=o)
                    g.capture_end()
                    for _ in range(3):
                        g.replay()
                    side.synchronize()
                    reps = 8
                    t0 = time.perf_counter()
                    for _ in range(reps):
                        g.replay()
                    side.synchronize()
                    return (time.perf_counter() - t0) / (reps * launches * wx.shape[1]) * 1e6

                one = replayed(wx1, o1, 64)
                many = replayed(wx16, o16, 16)
                dec.close()
                side.synchronize()
                graphs.clear()
            c = dec.control()
            assert not c["wait_expired"] and not c["collect_gave_up"], c
            out.append({"cell": f"{function} bf16 B{B} N{N} D{D}", "backend": "hip_fused, resident kernel",
                        "eager_us_per_token": eager, "graph_replay_us_per_token": one,
                        "graph_replay_us_per_token_16_per_post": many, "tokens_served": c["tokens_served"]})
    torch.cuda.current_stream().wait_stream(side)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="C2", choices=sorted(WORKLOADS) + ["C5s", "step"],
                    help="C1..C5: the benchmark configurations; C5s: the head-dim sweep of the fifth one on both backends; "
                         "step: single-step decoding latency")
    ap.add_argument("--shape", default=None, help="function:dtype:B:T:N:D, e.g. lstm:bfloat16:16:1024:1:768 (fwd+bwd, "
                    "zero initial state, cotangent on every state); replaces --workload")
    ap.add_argument("--backend", default=None, choices=["hip_fused", "hip"])
    ap.add_argument("--recompute", action="store_true",
                    help="hip_fused in recompute mode: no gate cache, the backward pass rebuilds the gates")
    ap.add_argument("--with-linear", action="store_true",
                    help="also time the step with the input projection Wx = Linear(x) in front (hidden size N*D)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-alt", action="store_true", help="skip the other-backend comparison leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain device-to-device copy of 256 MiB (a kernel of known traffic: 256 MiB read, "
                         "256 MiB written) so that a counter profile of this command holds its own calibration")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the recurrent path has no multi-GPU leg in this build "
              "(heads and batch rows shard without per-step communication); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (flashrnn_amd has no CPU path)", file=sys.stderr)
        sys.exit(2)
    device = torch.device("cuda:0")
    if args.shape:
        f, dt, B, T, N, D = args.shape.split(":")
        args.workload = "shape " + args.shape
        WORKLOADS[args.workload] = dict(function=f, dtype=dt, B=int(B), T=int(T), N=int(N), D=int(D), init="zeros",
                                        grad_on="all", bwd=True, seed=2000)
    if args.workload == "C5s":
        rows = run_sweep(device, args.steps, args.warmup)
        ref = rows[3]
        print(json.dumps({"metric": "tokens/s fwd+bwd, LSTM bf16 B16 T1024 head-dim sweep at N*D = 768 (fused vs alternating)",
                          "value": ref["tokens_per_s_hip_fused"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
                          "warmup": args.warmup, "ms_per_step": ref["hip_fused_ms"], "higher_is_better": True, "scaling": "weak",
                          "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                          "config": {"workload": "C5s: value and ms_per_step are the D = 256 point on hip_fused"}, "sweep": rows}))
        return
    if args.workload == "step":
        rows = run_steps(device)
        decode_rows = run_decode(device)
        ref = rows[0]
        print(json.dumps({"metric": "microseconds per single decoding step (flashrnn_step, fp32 carry)", "value": ref["graph_replay_us_per_step"],
                          "unit": "us/step", "n_gpus": 1, "steps": 256, "warmup": 20, "ms_per_step": ref["graph_replay_us_per_step"] / 1e3,
                          "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
                          "config": {"workload": "step: value is " + ref["cell"] + " on " + ref["backend"] + ", graph replay"},
                          "steps_table": rows, "resident_decode_table": decode_rows}))
        return
    w = WORKLOADS[args.workload]
    backend = args.backend or ("hip" if args.workload == "C5" else "hip_fused")
    tokens = w["B"] * w["T"]

    if args.copy_calibration:
        src = torch.arange(64 << 20, dtype=torch.float32, device=device)  # 256 MiB
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    ms, kern = run_gpu(w, backend, args.steps, args.warmup, device, recompute=args.recompute)

    # dominant kernel and its roofline: 2*N*G_r*D^2 flops per token in the forward scan and the
    # same in the reverse scan (dh = R^T dg) and in the dR GEMM
    flops_scan = 2.0 * w["N"] * GATES_R[w["function"]] * w["D"] ** 2 * tokens
    algo = {"fused_fwd_kernel": flops_scan, "fused_bwd_kernel": flops_scan, "grad_gemm_kernel": flops_scan,
            "alt_forward_steps": flops_scan, "alt_backward_steps": flops_scan}
    cand = {k: v for k, v in kern.items() if k in algo}
    dom = max(cand, key=lambda k: cand[k][0] * cand[k][1])
    dom_ms = cand[dom][0]
    peak = PEAK_TFLOPS[w["dtype"]]
    achieved = algo[dom] / cand[dom][1] / (dom_ms * 1e-3) / 1e12
    traffic, traffic_note = profiled_traffic(w, dom, args.recompute)
    roofline = dict(kernel=dom, bound="mfma", achieved=achieved, peak=peak, unit="TFLOP/s", frac=achieved / peak,
                    traffic=traffic, traffic_source=traffic_note, avg_launch_ms=dom_ms, launches_per_step=cand[dom][1],
                    us_per_time_step=dom_ms * 1e3 / w["T"])
    # the whole step against the same peak: 3 contractions of flops_scan each when there is a backward pass
    step_flops = flops_scan * (3.0 if w["bwd"] else 1.0)
    roofline.update(whole_step_tflops=step_flops / (ms * 1e-3) / 1e12, whole_step_frac=step_flops / (ms * 1e-3) / 1e12 / peak)
    try:
        from flashrnn_amd import fused_plan

        if backend == "hip_fused":
            wv, utw, kw, active = fused_plan(w["function"], w["dtype"], w["B"], w["N"], w["D"], dom == "fused_bwd_kernel")
            roofline.update(compute_units_used=active, wgs_per_head=kw,
                            frac_of_used_cus=achieved / (peak * active / 256.0))
    except Exception:  # plan query is informational only
        pass

    out = {
        "metric": "tokens/s fwd+bwd, LSTM bf16 B8 T1024 N3 D256; MFMA util vs peak" if args.workload == "C2"
                  else f"tokens/s {describe(w)}",
        "value": tokens / (ms * 1e-3), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": {"bfloat16": "bf16", "float16": "f16", "float32": "f32"}[w["dtype"]], "data": "synthetic",
        "config": {"workload": f"{args.workload}: {describe(w)}", "backend": backend, "seed": w["seed"],
                   "gate_cache": "recomputed in the backward pass" if args.recompute and backend == "hip_fused" else "stored",
                   "timed": "flashrnn() + torch.autograd.grad through the C ABI, inputs resident in HBM"},
        "roofline": roofline,
        "kernels_ms": {k: {"avg_ms": v[0], "per_step": v[1]} for k, v in kern.items()},
    }
    if not args.no_alt and w["bwd"]:
        other = "hip" if backend == "hip_fused" else "hip_fused"
        try:
            ms_o, _ = run_gpu(w, other, max(3, args.steps // 4), 2, device)
            out["other_backend"] = {"backend": other, "ms_per_step": ms_o, "tokens_per_s": tokens / (ms_o * 1e-3),
                                    "speedup_of_" + backend: ms_o / ms}
        except ValueError as e:  # no kernel of the other backend for this head dim
            out["other_backend"] = {"backend": other, "error": str(e)}
    if args.with_linear:
        ms_l = run_with_linear(w, backend, args.steps, args.warmup, device)
        out["with_linear"] = {"ms_per_step": ms_l, "linear_ms": ms_l - ms,
                              "note": "x [B,T,N*D] -> torch.nn.functional.linear -> view [B,T,G,N,D] -> flashrnn(); no copy in between"}
    if not args.no_cpu:
        out["cpu_baseline"] = run_cpu_baseline(w)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
