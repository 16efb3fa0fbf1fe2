#!/usr/bin/env python3
"""Benchmark of the fused fp8 LM-head + softcap + cross-entropy path on one MI355X.

A step is one forward + backward of the loss head over one batch of synthetic
input (resident in HBM before the timed region).  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload limited_2p7b]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0        # MI355X dense fp8 MFMA, published

PROFILE_KERNEL = {"fwd": "fwd_kernel", "recompute": "bwd_recompute_kernel", "dx": "bwd_dx_kernel<bf16_t, false>",
                  "dw": "bwd_dw_kernel<false>"}


def measured_traffic(workload, mode, kind):
    """HBM-side bytes per launch (fetched + written) of one kind of kernel, read from the committed rocprofv3
    counter summary of this very workload and mode (profiles/bench_<workload>_<mode>_pmc.txt: FETCH_SIZE / WRITE_SIZE
    scaled by a 1 GiB device copy), or None if there is none.  bench.py does not measure it itself: the counters need
    the profiler."""
    path = os.path.join(ROOT, "profiles", f"bench_{workload}_{mode}_pmc.txt")
    try:
        lines = open(path).read().splitlines()
    except OSError:
        return None
    name = PROFILE_KERNEL.get(kind)
    for ln in lines:
        if name and ln.startswith(name + " "):
            cols = ln[len(name):].split()
            try:
                return round((float(cols[1]) + float(cols[2])) * 2 ** 30)        # launches, fetched GiB/launch, written GiB/launch
            except (IndexError, ValueError):
                return None
    return None


def cpu_model():
    try:
        for ln in open("/proc/cpuinfo"):
            if ln.startswith("model name"):
                return ln.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(inp, rows, threads):
    """The eager reference path (oracle/eager.py) on the host cores, forward + backward,
    on the first `rows` rows against the full W."""
    import torch
    from oracle import eager
    x = inp.x[:rows].bfloat16()
    w = inp.w.bfloat16()
    y = inp.targets[:rows]
    t0 = time.time()
    eager.softcapped_ce(x, w, y, inp.x_s, inp.w_s, cap=inp.cap, reduction="mean", row_chunk=1024)
    dt = time.time() - t0
    return rows / dt, dt


class SocketPower:
    """The GPU's socket power (the hwmon sensor in sysfs, microwatts) sampled from a thread while something runs; every
    figure is None where the box has no such sensor."""

    def __init__(self, period=0.02):
        import glob
        self.path = next((f for f in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")) if self._read(f)), None)
        self.period, self.samples, self._stop, self._th = period, [], None, None

    @staticmethod
    def _read(path):
        try:
            return int(open(path).read()) * 1e-6
        except (OSError, ValueError):
            return None

    def __enter__(self):
        import threading
        if self.path:
            self._stop = threading.Event()

            def poll():
                while not self._stop.is_set():
                    v = self._read(self.path)
                    if v is not None:
                        self.samples.append(v)
                    time.sleep(self.period)

            self._th = threading.Thread(target=poll)
            self._th.start()
        return self

    def __exit__(self, *exc):
        if self._th:
            self._stop.set()
            self._th.join()

    def report(self):
        if not self.path or not self.samples:
            return None
        body = self.samples[len(self.samples) // 4:]          # the first quarter is the ramp
        cap = self._read(self.path.replace("power1_input", "power1_cap"))
        return {"sensor": "hwmon power1_input (socket)", "cap_w": None if cap is None else round(cap), "mean_w": round(sum(body) / len(body)),
                "max_w": round(max(body)), "samples": len(body),
                "during": "the pass with the per-kernel timers that follows the timed region (same steps)"}


def timed(step, steps, warmup=2):
    """ms per step over exactly `steps` steps, HIP events on torch's current stream (where the library launches)."""
    import torch
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / steps


def extras(args, inp, x, w, y, go, dev):
    """Further timings after the headline's timed region, each `extra_steps` steps of forward + backward: the other
    backward mode and the step with a weight cache at the headline workload, and the reference trainer's own call
    (tiny/train.py:682-696,1417-1419: N = 65536, d = 1024, three prediction offsets, fixed scales, per-row losses reduced
    with .mean()) through the autograd Function.  [{name, ms_per_step, frac_fp8_mfma_peak, ...}]"""
    import torch
    from slowrun_amd import configs
    from slowrun_amd import cuda_kernels as ck
    N, d, V = inp.shape
    out = []

    def entry(name, ms, n, dd, vv, **more):
        tf = 6.0 * n * dd * vv / (ms * 1e-3) * 1e-12
        e = {"name": name, "ms_per_step": round(ms, 4), "tokens_per_s": round(n / (ms * 1e-3), 1), "algorithmic_tflops": round(tf, 1),
             "frac_fp8_mfma_peak": round(tf / PEAK_FP8_TFLOPS, 4)}
        e.update(more)
        return e

    if args.rows is None and args.panel_rows == 0:
        other_keep = args.dlogits != "keep"

        def step_other():
            loss, saved, _l, _a, _n = ck.ce_forward(x, w, y, inp.x_s, inp.w_s, inp.cap, "mean", keep_dlogits=other_keep)
            ck.ce_backward(saved, y, go, N, d, V, inp.x_s, inp.w_s, inp.cap, 1.0, "mean", torch.bfloat16, torch.bfloat16, keep_dlogits=other_keep)

        ms = timed(step_other, args.extra_steps)
        out.append(entry(f"{inp.name}, dlogits {'kept' if other_keep else 'recomputed in backward (nothing N x V held)'}", ms, N, d, V,
                         hardware_flops_per_step=(6.0 if other_keep else 8.0) * N * d * V))
        keep = args.dlogits == "keep"
        cache = ck.WeightCache()

        def step_cached():
            loss, saved, _l, _a, _n = ck.ce_forward(x, w, y, inp.x_s, inp.w_s, inp.cap, "mean", keep_dlogits=keep, weight_cache=cache)
            ck.ce_backward(saved, y, go, N, d, V, inp.x_s, inp.w_s, inp.cap, 1.0, "mean", torch.bfloat16, torch.bfloat16, keep_dlogits=keep,
                           weight_cache=cache, cache_generation=cache.generation)

        ms = timed(step_cached, args.extra_steps)
        out.append(entry(f"{inp.name}, dlogits {args.dlogits}, W quantised once and cached across steps (a trainer's micro-steps "
                         "between optimizer steps)", ms, N, d, V))
        del cache
    # the trainer's call
    tin = configs.make_inputs("tiny_track", N=65536)
    tn, td, tv = tin.shape
    tx = tin.x.to(dev, torch.bfloat16).requires_grad_(True)
    tw = tin.w.to(dev, torch.bfloat16).requires_grad_(True)
    ty = tin.targets.to(dev)
    mw = torch.tensor([1.0, 0.5, 0.25], device=dev)

    def step_trainer():
        tx.grad = None
        tw.grad = None
        ck.FusedSoftcappedCrossEntropy.apply(tx, ty, mw, tw, 100 / 448, 1.6 / 448, 0.75 / 448, 1.0).mean().backward()

    ms = timed(step_trainer, args.extra_steps)
    out.append(entry(f"trainer call (tiny/train.py:694): N={tn}, d={td}, V={tv}, mtp_weights [1, 0.5, 0.25], x_s=100/448, w_s=1.6/448, "
                     "bf16 in, FusedSoftcappedCrossEntropy.apply(...).mean().backward()", ms, tn, td, tv))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="limited_2p7b")
    ap.add_argument("--rows", type=int, default=None, help="override N (debugging only; the result is then not the headline)")
    ap.add_argument("--panel-rows", type=int, default=0)
    ap.add_argument("--dlogits", choices=["keep", "recompute"], default="keep",
                    help="keep: the forward pass emits the dlogits (N x V bytes held until backward, backward is two GEMMs); "
                         "recompute: backward computes the logit tiles again (nothing N x V is held)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the further timings that follow the headline's timed region (the line's `other` list)")
    ap.add_argument("--extra-steps", type=int, default=10)
    ap.add_argument("--cpu-rows", type=int, default=16384)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="after the timed region, copy 1 GiB device to device once (a kernel of known traffic, "
                         "to scale rocprofv3's FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (one process, one MI355X); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from slowrun_amd import _lib, configs
    from slowrun_amd import cuda_kernels as ck

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    _lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    inp = configs.make_inputs(args.workload, N=args.rows)
    N, d, V = inp.shape
    x = inp.x.to(dev, torch.bfloat16)
    w = inp.w.to(dev, torch.bfloat16)
    y = inp.targets.to(dev)
    go = torch.ones((), device=dev)
    keep = args.dlogits == "keep"

    def step():
        loss, saved, _lse, _am, _nv = ck.ce_forward(x, w, y, inp.x_s, inp.w_s, inp.cap, "mean", keep_dlogits=keep)
        dx, dw = ck.ce_backward(saved, y, go, N, d, V, inp.x_s, inp.w_s, inp.cap, 1.0, "mean", torch.bfloat16, torch.bfloat16,
                                panel_rows=args.panel_rows, keep_dlogits=keep)
        return loss, dx, dw

    for _ in range(args.warmup):
        out = step()
    torch.cuda.synchronize()
    # timed region: exactly `steps` steps, no instrumentation
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.time()
    e0.record()
    for _ in range(args.steps):
        out = step()
    e1.record()
    torch.cuda.synchronize()
    wall = time.time() - t0
    ms_total = e0.elapsed_time(e1)
    # second pass of the same steps with the library's per-kernel HIP events switched on (roofline figures only)
    _lib.timing_enable(True)
    with SocketPower() as power:
        for _ in range(args.steps):
            out = step()
        torch.cuda.synchronize()
    kt = _lib.timing_read()
    _lib.timing_enable(False)
    ms_per_step = ms_total / args.steps
    loss = float(out[0])
    if args.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)      # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    other = []
    if not args.no_extras:
        other = extras(args, inp, x, w, y, go, dev)

    flops_step = 6.0 * N * d * V                      # algorithmic: logits + dX + dW, no recompute
    tokens_per_s = N / (ms_per_step * 1e-3)
    # per-kernel achieved rate: algorithmic flops of the launches of that kind / their time
    algo = {"fwd": 2.0 * N * d * V, "recompute": 2.0 * N * d * V, "dx": 2.0 * N * d * V, "dw": 2.0 * N * d * V}
    kernels = {}
    for k, (ms, n) in kt.items():
        if n == 0:
            continue
        per_step_ms = ms / args.steps
        ent = {"ms_per_step": round(per_step_ms, 4), "launches_per_step": n / args.steps, "avg_launch_ms": round(ms / n, 4)}
        if k in algo:
            ent["tflops"] = round(algo[k] / (per_step_ms * 1e-3) * 1e-12, 1)
        kernels[k] = ent
    dom = max((k for k in kernels if k in algo), key=lambda k: kernels[k]["ms_per_step"])
    roofline = {
        "bound": "mfma", "kernel": dom, "achieved": kernels[dom]["tflops"], "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
        "frac": round(kernels[dom]["tflops"] / PEAK_FP8_TFLOPS, 4),
        "traffic": (measured_traffic(args.workload, args.dlogits, dom) if (args.rows is None and args.panel_rows == 0) else None),
        "avg_launch_ms": kernels[dom]["avg_launch_ms"],
    }
    result = {
        "metric": "fp8 lm-head+softcap CE fwd+bwd tokens/s at d=2560,V=50304; % fp8 MFMA peak",
        "value": round(tokens_per_s, 1), "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "fp8_e4m3", "data": "synthetic",
        "config": {"workload": f"{inp.name}: N={N}, d={d}, V={V}, cap={inp.cap}, fp8 e4m3 amax scales, bf16 dX/dW, mean reduction",
                   "dlogits": ("kept from the forward pass (8 bits per logit held until backward)" if keep
                               else "recomputed in backward (nothing N x V held)"),
                   "argmax": "not asked for in the timed step (a debug output of the forward kernel, about 0.25 ms when asked for)",
                   "w_quantised": "every step, as the reference does (tiny/cuda_kernels.py:341-343); see `other` for the step with a weight cache"},
        "algorithmic_tflops": round(flops_step / (ms_per_step * 1e-3) * 1e-12, 1),
        "frac_fp8_mfma_peak": round(flops_step / (ms_per_step * 1e-3) * 1e-12 / PEAK_FP8_TFLOPS, 4),
        "hardware_flops_per_step": (6.0 if keep else 8.0) * N * d * V,
        "loss": loss,
        "wall_s_timed_region": round(wall, 3),
        "roofline": roofline,
        "kernels": kernels,
        "socket_power": power.report(),
        "other": other,
    }
    if not args.no_cpu_baseline:
        # every core this process has been given: torch's default thread count follows the OMP_NUM_THREADS the box sets
        # (its share of the host), not os.cpu_count(), which shows the whole machine
        threads = torch.get_num_threads()
        rows = min(args.cpu_rows, N)
        tps, dt = cpu_baseline(inp, rows, threads)
        result["cpu_baseline"] = {
            "value": round(tps, 1), "unit": "tokens/s", "cores": threads, "kind": "port",
            "host_cpus": os.cpu_count(), "cpu_model": cpu_model(), "torch_threads": threads,
            "sample": f"eager fp8-quantise + fp32 matmul + softcap + F.cross_entropy fwd+bwd on the first {rows} rows "
                      f"against the full (d,V) weight, {dt:.1f} s, torch {torch.__version__} with {threads} threads",
        }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
