"""What the MI355X in front of us sustains on fp8 matrix work, measured: ``python -m slowrun_amd.ceiling``.

The loss head is bound by the matrix pipe, whose published peak (5.0 PFLOP/s dense fp8) assumes the full 2.4 GHz
shader clock.  This report puts numbers beside that peak, each from a short run on the GPU at hand:

  1. the matrix instruction alone (operands in registers), on constant and on random operands, with the shader clock
     the kernel itself saw;
  2. the library's main loop alone (global -> LDS -> MFMA, no epilogue) on the three GEMM shapes of the headline
     workload, on random and on all-zero operands;
  3. the vendor library's fp8 GEMM (torch._scaled_mm -> hipBLASLt) on the same shapes;
  4. the three big kernels of a step and their main loops alone on the step's own operands;
  5. the socket power (sysfs) and the shader clock (rocm-smi) while the main loop runs flat out, on random and on
     all-zero operands.

Prints a plain-text report (and one JSON line at the end).  Nothing here is on the product path.
"""
import argparse
import ctypes as C
import json
import subprocess
import threading
import time

import torch

from . import _lib

PEAK_FP8_TFLOPS = 5000.0


def _mfma(random, scratch, iters=20000, reps=3):
    dev = scratch.device
    data = None
    if random:
        ncu = torch.cuda.get_device_properties(dev).multi_processor_count
        data = torch.randint(0, 256, (4 * ncu * 65536,), dtype=torch.uint8, device=dev)
        data[(data & 0x7f) == 0x7f] = 0x38                          # no NaN codes among the operands
    tf, mhz = C.c_double(), C.c_double()
    _lib.check(_lib.lib().sce_bench_mfma(data.data_ptr() if random else None, data.numel() if random else 0, iters, reps, scratch.data_ptr(), scratch.numel(),
                                         dev.index, None, C.byref(tf), C.byref(mhz)), "sce_bench_mfma")
    return tf.value, mhz.value


def _operand(rows, K, kind, dev):
    t = torch.zeros(rows, K + 128, dtype=torch.uint8, device=dev)
    if kind == "random":
        v = torch.randint(0, 256, (rows, K), dtype=torch.uint8, device=dev)
        v[(v & 0x7f) == 0x7f] = 0x38
        t[:, :K] = v
    return t


def _gemm(M, N, K, kind, scratch, reps=5):
    dev = scratch.device
    a, b = _operand(M, K, kind, dev), _operand(N, K, kind, dev)
    tf, mhz = C.c_double(), C.c_double()
    _lib.check(_lib.lib().sce_bench_gemm(a.data_ptr(), b.data_ptr(), M, N, K, reps, scratch.data_ptr(), scratch.numel(), dev.index,
                                         None, C.byref(tf), C.byref(mhz)), "sce_bench_gemm")
    return tf.value, mhz.value


def _hipblaslt(M, N, K, dev, reps=5):
    """The vendor's GEMM on the very bytes section 2 uses (uniformly random, no NaN codes), so that the two sections
    differ in the kernel and not in how often the operand bits toggle."""
    a = _operand(M, K, "random", dev)[:, :K].contiguous().view(torch.float8_e4m3fn)
    b = _operand(N, K, "random", dev)[:, :K].contiguous().view(torch.float8_e4m3fn)
    one = torch.ones((), device=dev)
    try:
        f = lambda: torch._scaled_mm(a, b.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)
        f()
    except Exception as e:                      # noqa: BLE001 - reported, not fatal
        return None, str(e).splitlines()[0]
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        f()
    e1.record()
    torch.cuda.synchronize()
    return 2.0 * M * N * K * reps / (e0.elapsed_time(e1) * 1e-3) * 1e-12, None


def _hwmon():
    """The GPU's power sensor in sysfs (socket power in microwatts, and its cap), if the box exposes one."""
    import glob
    for f in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input")):
        try:
            open(f).read()
            return f
        except OSError:
            continue
    return None


def _power_w(sensor):
    try:
        return round(int(open(sensor).read()) * 1e-6)
    except (OSError, ValueError, TypeError):
        return None


def _smi_sample(sensor=None):
    try:
        out = subprocess.run(["rocm-smi", "--showclocks", "--json"], capture_output=True, text=True, timeout=10).stdout
        card = next(iter(json.loads(out).values()))
    except Exception:                            # noqa: BLE001
        return None
    sclk = next((v for k, v in card.items() if "sclk" in k.lower()), None)
    return {"sclk": sclk, "power_w": _power_w(sensor)}


def _under_load(scratch, kind, sensor, seconds=4.0):
    """Socket power (sysfs) and rocm-smi's shader clock while the main loop runs on `kind` operands."""
    dev = scratch.device
    a, b = _operand(8192, 8192, kind, dev), _operand(8192, 8192, kind, dev)
    samples, stop = [], threading.Event()

    def poll():
        while not stop.is_set():
            smp = _smi_sample(sensor)
            if smp:
                samples.append(smp)
            time.sleep(0.3)

    th = threading.Thread(target=poll)
    th.start()
    tf, mhz = C.c_double(), C.c_double()
    t0 = time.time()
    rates = []
    while time.time() - t0 < seconds:
        _lib.check(_lib.lib().sce_bench_gemm(a.data_ptr(), b.data_ptr(), 8192, 8192, 8192, 40, scratch.data_ptr(), scratch.numel(),
                                             dev.index, None, C.byref(tf), C.byref(mhz)), "sce_bench_gemm")
        rates.append((tf.value, mhz.value))
    stop.set()
    th.join()
    return samples, rates


def _floor(workload, scratch, reps=5, sensor=None):
    """One forward (dlogits kept) + backward of `workload`, timed per kernel kind by the library's events; then the main loops
    of the three big kernels alone (sce_bench_floor) on the buffers those calls left, and on all-zero buffers of the same
    sizes.  Returns {kind: {kernel_ms, floor_ms, floor_mhz, floor_zero_ms, floor_zero_mhz}}."""
    from . import configs
    from . import cuda_kernels as ck
    inp = configs.make_inputs(workload)
    N, d, V = inp.shape
    dev = scratch.device
    x, w, y = inp.x.to(dev, torch.bfloat16), inp.w.to(dev, torch.bfloat16), inp.targets.to(dev)
    sz = _lib.sizes_for(N, d, V)
    saved = torch.empty(sz.saved_bytes + sz.dlogits_bytes, dtype=torch.uint8, device=dev)
    fws = torch.empty(sz.fwd_workspace_bytes, dtype=torch.uint8, device=dev)
    bws = torch.empty(sz.bwd_workspace_kept_bytes, dtype=torch.uint8, device=dev)
    loss = torch.empty(1, dtype=torch.float32, device=dev)
    nv = torch.empty(2, dtype=torch.int32, device=dev)
    go = torch.ones(1, dtype=torch.float32, device=dev)
    dx = torch.empty(N, d, dtype=torch.bfloat16, device=dev)
    dw = torch.empty(d, V, dtype=torch.bfloat16, device=dev)
    a = ck._base_args(x, N, d, V, inp.x_s, inp.w_s, inp.cap, 1.0, "mean", y)
    a.x, a.x_dtype, a.x_ld = x.data_ptr(), _lib.SCE_BF16, d
    a.w, a.w_dtype, a.w_ld = w.data_ptr(), _lib.SCE_BF16, V
    a.loss, a.n_valid = loss.data_ptr(), nv.data_ptr()
    a.saved, a.saved_bytes = saved.data_ptr(), saved.numel()
    a.dlogits_from_forward = 1
    a.grad_output = go.data_ptr()
    a.dx, a.dx_dtype, a.dx_ld = dx.data_ptr(), _lib.SCE_BF16, d
    a.dw, a.dw_dtype, a.dw_ld = dw.data_ptr(), _lib.SCE_BF16, V

    def step():
        a.workspace, a.workspace_bytes = fws.data_ptr(), fws.numel()
        _lib.check(_lib.lib().sce_forward(C.byref(a)), "sce_forward")
        a.workspace, a.workspace_bytes = bws.data_ptr(), bws.numel()
        _lib.check(_lib.lib().sce_backward(C.byref(a)), "sce_backward")

    for _ in range(2):
        step()
    torch.cuda.synchronize()
    _lib.timing_enable(True)
    for _ in range(reps):
        step()
    torch.cuda.synchronize()
    kt = _lib.timing_read()
    _lib.timing_enable(False)
    kinds = {"fwd": 1, "dx": 5, "dw": 6}          # SCE_K_FWD, SCE_K_DX, SCE_K_DW
    out = {k: {"kernel_ms": round(kt[k][0] / reps, 3)} for k in kinds}
    flops = 2.0 * N * d * V

    def floors(tag):
        for k, which in kinds.items():
            ms, mhz = C.c_double(), C.c_double()
            _lib.check(_lib.lib().sce_bench_floor(C.byref(a), which, reps, scratch.data_ptr(), scratch.numel(), C.byref(ms), C.byref(mhz)),
                       "sce_bench_floor")
            out[k][tag + "_ms"], out[k][tag + "_mhz"] = round(ms.value, 3), round(mhz.value)

    floors("floor")
    saved.zero_()
    bws.zero_()
    floors("floor_zero")
    for k in kinds:
        r = out[k]
        print(f"   {k:3s}: kernel {r['kernel_ms']:6.3f} ms = {flops / r['kernel_ms'] * 1e-9:6.0f} TFLOP/s | main loop alone on the same operands "
              f"{r['floor_ms']:6.3f} ms = {flops / r['floor_ms'] * 1e-9:6.0f} TFLOP/s at {r['floor_mhz']:4d} MHz | on all-zero operands "
              f"{r['floor_zero_ms']:6.3f} ms = {flops / r['floor_zero_ms'] * 1e-9:6.0f} TFLOP/s at {r['floor_zero_mhz']:4d} MHz")
    tot_k, tot_f = sum(out[k]["kernel_ms"] for k in kinds), sum(out[k]["floor_ms"] for k in kinds)
    print(f"   sum: kernels {tot_k:.3f} ms, main loops alone {tot_f:.3f} ms = {3 * flops / tot_f * 1e-9 / PEAK_FP8_TFLOPS * 100:.1f} % of peak "
          "for a step that did nothing else")
    power = None
    if sensor:                                   # last, so that the timings above are of a part as cool as bench.py finds it: socket power while steps run back to back
        pw, stop = [], threading.Event()

        def poll():
            while not stop.is_set():
                pw.append(_power_w(sensor))
                time.sleep(0.05)

        th = threading.Thread(target=poll)
        th.start()
        t0, nsteps = time.time(), 0
        torch.cuda.synchronize()
        while time.time() - t0 < 3.0:
            for _ in range(10):
                step()
            torch.cuda.synchronize()
            nsteps += 10
        sustained_ms = (time.time() - t0) * 1e3 / nsteps
        stop.set()
        th.join()
        pw = [v for v in pw[len(pw) // 4:] if v is not None]          # the first quarter is the ramp
        if pw:
            power = {"mean_w": round(sum(pw) / len(pw)), "max_w": max(pw), "min_w": min(pw), "steps": nsteps, "ms_per_step": round(sustained_ms, 3)}
    if power:
        out["step_power"] = power
        print(f"   socket power while {power['steps']} such steps run back to back ({power['ms_per_step']} ms each by the host's clock): "
              f"mean {power['mean_w']} W, {power['min_w']} - {power['max_w']} W")
    del saved, fws, bws
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--no-smi", action="store_true")
    args = ap.parse_args()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    scratch = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
    rep = {"peak_fp8_tflops": PEAK_FP8_TFLOPS}
    print(f"device: {torch.cuda.get_device_name(dev)}; published dense fp8 peak {PEAK_FP8_TFLOPS:.0f} TFLOP/s at 2400 MHz")
    print("\n1. v_mfma_f32_32x32x64_f8f6f4 alone (operands in registers, 16 independent accumulators per wave)")
    rep["mfma_only"] = {}
    for kind in ("constant", "random"):
        tf, mhz = _mfma(kind == "random", scratch)
        rep["mfma_only"][kind] = {"tflops": round(tf, 1), "shader_mhz": round(mhz)}
        print(f"   {kind:9s} operands: {tf:7.1f} TFLOP/s = {tf / PEAK_FP8_TFLOPS * 100:5.1f} % of peak, shader clock seen by the kernel {mhz:5.0f} MHz")
    print("\n2. the main loop alone (global -> LDS -> MFMA, sums of the accumulators stored)")
    shapes = [("square", 8192, 8192, 8192), ("logits  (V x N, K = d)", 50432, 65536, 2560), ("dX      (d x N, K = V)", 2560, 65536, 50432),
              ("dW      (d x V, K = N)", 2560, 50432, 65536)]
    rep["main_loop"] = {}
    for name, M, N, K in shapes:
        row = {}
        for kind in ("random", "zero"):
            tf, mhz = _gemm(M, N, K, kind, scratch, reps=3 if M * N * K > 1e12 else 10)
            row[kind] = {"tflops": round(tf, 1), "shader_mhz": round(mhz)}
        rep["main_loop"][name.split()[0]] = row
        print(f"   {name:24s} random operands {row['random']['tflops']:7.1f} TFLOP/s at {row['random']['shader_mhz']:4d} MHz | "
              f"all-zero operands {row['zero']['tflops']:7.1f} TFLOP/s at {row['zero']['shader_mhz']:4d} MHz")
    print("\n3. torch._scaled_mm (hipBLASLt) fp8 e4m3, bf16 out, the same random operand bytes")
    rep["hipblaslt"] = {}
    for name, M, N, K in shapes:
        tf, err = _hipblaslt(N, M, K, dev, reps=3 if M * N * K > 1e12 else 10)
        rep["hipblaslt"][name.split()[0]] = None if tf is None else round(tf, 1)
        print(f"   {name:24s} " + (f"{tf:7.1f} TFLOP/s" if tf is not None else f"not available: {err}"))
    print("\n4. the three big kernels of a step and their main loops alone, on the step's own operand buffers (limited_2p7b: N = 65536, d = 2560, V = 50304)")
    sensor = None if args.no_smi else _hwmon()
    rep["floor"] = _floor("limited_2p7b", scratch, sensor=sensor)
    if not args.no_smi:
        cap = None
        if sensor:
            try:
                cap = round(int(open(sensor.replace("power1_input", "power1_cap")).read()) * 1e-6)
            except (OSError, ValueError):
                pass
        print(f"\n5. socket power (sysfs hwmon, cap {cap} W) and rocm-smi's shader clock while the main loop runs (8192^3)")
        idle = _smi_sample(sensor)
        print(f"   idle: {idle}")
        rep["smi"] = {"cap_w": cap, "idle": idle}
        for kind in ("random", "zero"):
            samples, rates = _under_load(scratch, kind, sensor)
            pick = lambda v: v[:: max(1, len(v) // 6)]
            rep["smi"][kind] = {"samples": pick(samples), "tflops": pick([round(r[0], 1) for r in rates]), "shader_mhz": pick([round(r[1]) for r in rates])}
            print(f"   {kind} operands:")
            for smp in rep["smi"][kind]["samples"]:
                print(f"      {smp}")
            print(f"      main loop meanwhile: {rep['smi'][kind]['tflops']} TFLOP/s at {rep['smi'][kind]['shader_mhz']} MHz (in-kernel)")
    print("\n" + json.dumps(rep))


if __name__ == "__main__":
    main()
