"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu-baseline]

A step is one launch of the workload's kernel through ``ninetoothed_amd.make``
(i.e. through the C ABI of libnt_hip.so) on synthetic, seeded inputs that are
already resident in HBM.  The default workload is the one the headline metric
is quoted on: addmm, fp16, M = N = K = 8192, alpha = 1.0, beta = 0.5.  The other
configurations of the baseline (512^3 matmul, 4096^2 fp32 softmax, SDPA forward
[4, 32, 4096, 128] causal / non-causal, conv2d [32, 256, 56, 56] * [256, 256, 3, 3])
are measured in the same run and reported under ``"others"``.

Prints ONE JSON line.  ``roofline.achieved`` = algorithmic FLOP (or bytes) per
launch / average launch time from device events on the launch stream.
``cpu_baseline`` times the CPU oracle (oracle/programs.py, single thread) on a
bounded sample of the same workload; ``torch_cpu`` times the stock torch CPU
operator of every configuration (all host threads, bounded samples);
``triton_interpreter_cpu`` times the 512^3 matmul as the reference runs on a CPU: a Triton kernel
under ``TRITON_INTERPRET=1`` (one thread).  ``vendor_gpu`` times the stock PyTorch
operator of each workload (hipBLASLt / MIOpen / the built-in SDPA) on the same
GPU and inputs, for context only.

The GPU clock needs a few milliseconds of load to settle, so the default warm-up
is 25 launches and the timed region 50.
"""

import argparse
import json
import os
import sys
import time

PEAK_TFLOPS = 2500.0  # dense fp16 MFMA, MI355X
PEAK_GBS = 8000.0     # HBM3E, MI355X

METRIC = "TFLOP/s fp16 matmul 8192^3 + attention fwd on 1 MI355X; % of MFMA peak"


def parse_args():
    parser = argparse.ArgumentParser()
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=50)
    parser.add_argument("--warmup", type=int, default=25)
    parser.add_argument("--workload", default="addmm_8192")
    parser.add_argument("--only", action="store_true", help="measure only --workload")
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-vendor", action="store_true", help="skip the stock PyTorch operators")
    parser.add_argument("--inputs", choices=("randn", "constant"), default="randn",
                        help="`constant` fills every tensor with one value instead of the seeded normal values the metric is quoted on: "
                             "the matrix pipe then draws far less power and the part keeps its clock (a diagnostic, never the reported figure)")
    return parser.parse_args()


def build_workloads(inputs="randn"):
    import torch

    import ninetoothed_amd as ninetoothed
    from ninetoothed_amd import programs

    def seeded(*shape, dtype=torch.float16, scale=1.0, seed=0):
        if inputs == "constant":
            return torch.full(shape, 0.5 * scale, dtype=dtype)
        generator = torch.Generator().manual_seed(seed)
        return (torch.randn(*shape, generator=generator) * scale).to(dtype)

    workloads = {}

    def addmm_8192():
        n = 8192
        input, mat1, mat2 = (seeded(n, n, seed=s).cuda() for s in (0, 1, 2))
        out = torch.empty(n, n, dtype=torch.float16, device="cuda")
        kernel = ninetoothed.make(programs.addmm.arrangement, programs.addmm.application, programs.addmm.tensors())
        return dict(
            step=lambda: kernel(input, mat1, mat2, 0.5, 1.0, out),
            vendor=lambda: torch.addmm(input, mat1, mat2, beta=0.5, alpha=1.0, out=out),
            work=2.0 * n**3, bound="mfma", kernel=kernel,
            describe={"workload": "addmm fp16 M=N=K=8192 alpha=1.0 beta=0.5", "inputs": "randn, seeded"},
        )

    def matmul_512():
        n = 512
        a, b = seeded(n, n, seed=0).cuda(), seeded(n, n, seed=1).cuda()
        out = torch.empty(n, n, dtype=torch.float16, device="cuda")
        kernel = ninetoothed.make(programs.matmul.arrangement, programs.matmul.application, programs.matmul.tensors())
        return dict(step=lambda: kernel(a, b, out), vendor=lambda: torch.matmul(a, b, out=out), work=2.0 * n**3, bound="mfma", kernel=kernel,
                    describe={"workload": "matmul fp16 M=N=K=512 (README program)"})

    def softmax_4096():
        x = seeded(4096, 4096, dtype=torch.float32).cuda()
        out = torch.empty_like(x)
        kernel = ninetoothed.make(programs.softmax.arrangement, programs.softmax.application, programs.softmax.tensors())
        return dict(step=lambda: kernel(x, out, BLOCK_SIZE=4096), vendor=lambda: torch.softmax(x, dim=-1, out=out), work=2.0 * 4096 * 4096 * 4, bound="hbm", kernel=kernel,
                    describe={"workload": "row softmax fp32 [4096, 4096]"})

    def attention(is_causal):
        def make():
            q, k, v = (seeded(4, 32, 4096, 128, seed=s).cuda() for s in (0, 1, 2))
            o = torch.empty_like(q)
            kernel = ninetoothed.make(programs.attention.arrangement_with_scale, programs.attention.application_with_scale, programs.attention.tensors(True))
            flops = 4.0 * 4 * 32 * 4096 * 4096 * 128 * (0.5 if is_causal else 1.0)
            return dict(step=lambda: kernel(q, k, v, is_causal, 128**-0.5, o),
                        vendor=lambda: torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=is_causal, scale=128**-0.5),
                        work=flops, bound="mfma", kernel=kernel,
                        describe={"workload": f"SDPA forward fp16 [4, 32, 4096, 128] scale=1/sqrt(128) causal={is_causal}"})
        return make

    def conv2d():
        x = seeded(32, 256, 56, 56, scale=0.1, seed=0).cuda()
        w = seeded(256, 256, 3, 3, scale=0.1, seed=1).cuda()
        out = torch.empty(32, 256, 56, 56, dtype=torch.float16, device="cuda")
        kernel = ninetoothed.make(programs.conv2d.arrangement, programs.conv2d.application, programs.conv2d.tensors())
        return dict(step=lambda: kernel(x, w, out, padding_h=1, padding_w=1), vendor=lambda: torch.nn.functional.conv2d(x, w, padding=1), work=2.0 * (32 * 56 * 56) * 256 * (256 * 9), bound="mfma", kernel=kernel,
                    describe={"workload": "conv2d fp16 x[32,256,56,56] w[256,256,3,3] stride 1 padding 1 (implicit GEMM)"})

    def map_add():
        # an element-wise program outside the five recognised ones: runs on the interpreter kernel
        n = 1 << 26
        lhs, rhs = seeded(n, dtype=torch.float32, seed=0).cuda(), seeded(n, dtype=torch.float32, seed=1).cuda()
        out = torch.empty_like(lhs)
        block = ninetoothed.Symbol("BLOCK_SIZE", meta=True)

        def arrangement(lhs, rhs, output):
            return lhs.tile((block,)), rhs.tile((block,)), output.tile((block,))

        def application(lhs, rhs, output):
            output = lhs + rhs  # noqa: F841

        kernel = ninetoothed.make(arrangement, application, (ninetoothed.Tensor(1),) * 3)
        return dict(step=lambda: kernel(lhs, rhs, out), vendor=lambda: torch.add(lhs, rhs, out=out), work=3.0 * n * 4, bound="hbm", kernel=kernel,
                    describe={"workload": "element-wise add fp32, 2^26 elements (generic tile-map executor)"})

    def copy_1gib():
        # a plain device-to-device copy of known size: the calibration point for the
        # HBM traffic counters (FETCH_SIZE / WRITE_SIZE) quoted in profiles/
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)

        class _Copy:
            last_plan = "torch copy_ (not part of the library)"

        return dict(step=lambda: dst.copy_(src), work=2.0 * (1 << 30), bound="hbm", kernel=_Copy(),
                    describe={"workload": "device copy of 1 GiB (2 GiB of traffic), counter calibration only"})

    def mfma_ceiling(constant, form="32x32x16"):
        # not a program of the library: MFMAs on register operands taken from the addmm workload's own inputs
        # (or from constants), which bounds what the GEMM and attention kernels can reach on this data
        def make():
            import ctypes

            from ninetoothed_amd import runtime

            n = 8192
            if constant:
                mat1, mat2 = (torch.full((n, n), 0.5, dtype=torch.float16, device="cuda") for _ in range(2))
            else:
                mat1, mat2 = (seeded(n, n, seed=s).cuda() for s in (1, 2))
            sink = torch.zeros(1, device="cuda")
            loops = 4096
            count = ctypes.c_int64(0)
            lib = load_probe_library()
            probe = lib.nt_probe_mfma_rate if form == "32x32x16" else lib.nt_probe_mfma_rate_16x16x32
            flop_per_mfma = 2 * 32 * 32 * 16 if form == "32x32x16" else 2 * 16 * 16 * 32

            def step():
                runtime.check(probe(runtime.current_stream(), runtime.ArgumentTensor.from_torch_tensor(mat1), runtime.ArgumentTensor.from_torch_tensor(mat2),
                                    loops, sink.data_ptr(), ctypes.byref(count)))

            step()

            class _Probe:
                last_plan = ("nt_probe_mfma_rate" if form == "32x32x16" else "nt_probe_mfma_rate_16x16x32") + " (measurement aid, not a program)"

            return dict(step=step, work=float(count.value) * flop_per_mfma, bound="mfma", kernel=_Probe(),
                        describe={"workload": "MFMA " + form + " fp16 issue rate on register operands, " + ("constant 0.5" if constant else "the addmm workload's N(0,1) inputs")})
        return make

    workloads["addmm_8192"] = addmm_8192
    workloads["mfma_ceiling"] = mfma_ceiling(False)
    workloads["mfma_ceiling_constant"] = mfma_ceiling(True)
    workloads["mfma_ceiling_16x16x32"] = mfma_ceiling(False, "16x16x32")  # the form the GEMM kernel issues
    workloads["matmul_512"] = matmul_512
    workloads["softmax_4096"] = softmax_4096
    workloads["attention"] = attention(False)
    workloads["attention_causal"] = attention(True)
    workloads["conv2d"] = conv2d
    workloads["map_add"] = map_add
    workloads["copy_1gib"] = copy_1gib
    return workloads


def load_probe_library():
    """``libnt_probe.so``: the MFMA issue-rate kernels (measurement aids, built beside the product library and
    loaded by nothing else)."""
    import ctypes

    from ninetoothed_amd import runtime
    from ninetoothed_amd.build_library import PROBE_LIBRARY_PATH

    if not PROBE_LIBRARY_PATH.exists():
        raise RuntimeError(f"{PROBE_LIBRARY_PATH} is missing: build it with `python -m ninetoothed_amd.build_library`")
    lib = ctypes.CDLL(str(PROBE_LIBRARY_PATH))
    for name in ("nt_probe_mfma_rate", "nt_probe_mfma_rate_16x16x32"):
        function = getattr(lib, name)
        function.argtypes = [ctypes.c_void_p, runtime.ArgumentTensor, runtime.ArgumentTensor, ctypes.c_int, ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64)]
        function.restype = ctypes.c_int
    return lib


def launch_description(workload):
    """The prepared launch of the workload's latest call plus the kernel variant the library ran for it."""
    from ninetoothed_amd import runtime

    plan = workload["kernel"].last_plan
    if not str(plan).startswith("launch_nt_"):
        return plan
    return f"{plan}; {runtime.last_launch()}"


def measure(workload, steps, warmup, which="step"):
    """Times exactly ``steps`` launches with device events on the launch stream."""
    import torch

    workload = {"step": workload[which]}
    for _ in range(warmup):
        workload["step"]()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    wall0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        workload["step"]()
    stop.record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - wall0) * 1e3 / steps
    device_ms = start.elapsed_time(stop) / steps
    return device_ms, wall


def per_launch(workload, launches=20):
    """Median and minimum of single launches, each bracketed by its own pair of events."""
    import torch

    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(launches)]
    for start, stop in events:
        start.record()
        workload["step"]()
        stop.record()
    torch.cuda.synchronize()
    times = sorted(start.elapsed_time(stop) for start, stop in events)
    return {"median_ms": times[len(times) // 2], "min_ms": times[0], "launches": launches}


def roofline(workload, device_ms, traffic):
    if workload["bound"] == "mfma":
        achieved = workload["work"] / (device_ms * 1e-3) / 1e12
        return {"bound": "mfma", "achieved": achieved, "peak": PEAK_TFLOPS, "unit": "TFLOP/s", "frac": achieved / PEAK_TFLOPS, "traffic": traffic}
    achieved = workload["work"] / (device_ms * 1e-3) / 1e9
    return {"bound": "hbm", "achieved": achieved, "peak": PEAK_GBS, "unit": "GB/s", "frac": achieved / PEAK_GBS, "traffic": traffic}


def cpu_baseline_addmm():
    """The CPU oracle (tile-by-tile numpy restatement) on a 512-row band of the
    8192^3 addmm: 512 x 8192 x 8192, one thread."""
    import numpy as np
    from threadpoolctl import threadpool_limits

    from oracle import programs as oracle

    rows, n = 512, 8192
    rng = np.random.default_rng(0)
    input = rng.standard_normal((rows, n), dtype=np.float32).astype(np.float16)
    mat1 = rng.standard_normal((rows, n), dtype=np.float32).astype(np.float16)
    mat2 = rng.standard_normal((n, n), dtype=np.float32).astype(np.float16)
    with threadpool_limits(limits=1):
        t0 = time.perf_counter()
        oracle.addmm(input, mat1, mat2, 0.5, 1.0, bm=64, bn=64, bk=64)
        seconds = time.perf_counter() - t0
    flops = 2.0 * rows * n * n
    return {
        "value": flops / seconds / 1e12,
        "unit": "TFLOP/s",
        "cores": 1,
        "kind": "port",
        "sample": f"oracle.addmm on a {rows}x{n}x{n} band of the workload (64x64x64 blocks), {seconds:.1f} s",
    }


def triton_interpreter_cpu():
    """The reference's CPU path for the 512^3 matmul: a Triton kernel with the structure of the one the
    reference generates, run by Triton's interpreter (oracle/triton_cpu_matmul.py), in a process of its
    own because the interpreter switch has to be set before Triton is imported.  The child uses CPU
    tensors only."""
    import subprocess

    root = os.path.dirname(os.path.abspath(__file__))
    env = dict(os.environ, TRITON_INTERPRET="1")
    try:
        done = subprocess.run([sys.executable, "-m", "oracle.triton_cpu_matmul", "512"], cwd=root, env=env, capture_output=True, text=True, timeout=600)
        lines = [line for line in done.stdout.splitlines() if line.startswith("{")]
        if done.returncode != 0 or not lines:
            return {"error": (done.stderr or done.stdout).strip().splitlines()[-1][:200] if (done.stderr or done.stdout).strip() else f"exit code {done.returncode}"}
        result = json.loads(lines[-1])
    except Exception as error:
        return {"error": str(error)[:200]}
    if "error" not in result:
        result["kind"] = "own Triton kernel of the reference's structure under TRITON_INTERPRET=1"
        result["workload"] = "matmul fp16 M=N=K=512"
    return result


def torch_cpu_context():
    """The stock torch CPU operator of each configuration on the host, all threads,
    one warm-up and the median of three runs, on bounded samples (context only)."""
    import torch
    import torch.nn.functional as F

    generator = torch.Generator().manual_seed(0)

    def randn(*shape, scale=1.0):
        return torch.randn(*shape, generator=generator) * scale

    def timed(fn, runs=3, warm=1):
        for _ in range(warm):
            fn()
        times = []
        for _ in range(runs):
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        return sorted(times)[len(times) // 2]

    out = {"threads": torch.get_num_threads(), "host_cpus": os.cpu_count()}
    rows, n = 1024, 8192
    input, mat1, mat2 = randn(rows, n), randn(rows, n), randn(n, n)
    seconds = timed(lambda: torch.addmm(input, mat1, mat2, beta=0.5, alpha=1.0), runs=1, warm=0)
    out["addmm_8192"] = {"value": 2.0 * rows * n * n / seconds / 1e12, "unit": "TFLOP/s", "sample": f"torch.addmm fp32 on a {rows}x{n}x{n} band, {seconds:.2f} s"}
    a, b = randn(512, 512), randn(512, 512)
    seconds = timed(lambda: torch.matmul(a, b))
    out["matmul_512"] = {"value": 2.0 * 512**3 / seconds / 1e12, "unit": "TFLOP/s", "sample": f"torch.matmul fp32 512^3, {seconds * 1e3:.2f} ms"}
    x = randn(4096, 4096)
    seconds = timed(lambda: torch.softmax(x, dim=-1))
    out["softmax_4096"] = {"value": 2.0 * 4096 * 4096 * 4 / seconds / 1e9, "unit": "GB/s", "sample": f"torch.softmax fp32 [4096, 4096], {seconds * 1e3:.1f} ms"}
    q, k, v = (randn(1, 2, 4096, 128) for _ in range(3))
    for causal, name in ((False, "attention"), (True, "attention_causal")):
        seconds = timed(lambda: F.scaled_dot_product_attention(q, k, v, is_causal=causal, scale=128**-0.5), runs=1, warm=0)
        flops = 4.0 * 2 * 4096 * 4096 * 128 * (0.5 if causal else 1.0)
        out[name] = {"value": flops / seconds / 1e12, "unit": "TFLOP/s", "sample": f"F.scaled_dot_product_attention fp32 on 2 of the 128 (batch, head) pairs, {seconds:.2f} s"}
    xc, wc = randn(2, 256, 56, 56, scale=0.1), randn(256, 256, 3, 3, scale=0.1)
    seconds = timed(lambda: F.conv2d(xc, wc, padding=1), runs=1, warm=0)
    out["conv2d"] = {"value": 2.0 * (2 * 56 * 56) * 256 * (256 * 9) / seconds / 1e12, "unit": "TFLOP/s", "sample": f"F.conv2d fp32 on 2 of the 32 images, {seconds:.2f} s"}
    return out


def load_traffic():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", "hbm_traffic.json")
    if os.path.exists(path):
        with open(path) as handle:
            return json.load(handle)
    return {}


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: this build has no multi-GPU path (asked for --gpus {args.gpus}).", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU path).", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)

    workloads = build_workloads(args.inputs)
    if args.workload not in workloads:
        print(f"unknown workload `{args.workload}`; choose from {sorted(workloads)}", file=sys.stderr)
        sys.exit(2)
    traffic = load_traffic()

    main_workload = workloads[args.workload]()
    device_ms, wall_ms = measure(main_workload, args.steps, args.warmup)
    main_roofline = roofline(main_workload, device_ms, traffic.get(args.workload))
    launch_plan = launch_description(main_workload)
    single = per_launch(main_workload)
    vendor = {}

    def vendor_line(name, workload, steps):
        if args.no_vendor or "vendor" not in workload:
            return
        try:
            ms, _ = measure(workload, steps, args.warmup, which="vendor")
        except Exception as error:  # a stock operator that is missing on this build is not this library's failure
            vendor[name] = {"error": str(error).splitlines()[0][:120]}
            return
        entry = roofline(workload, ms, None)
        vendor[name] = {"achieved": entry["achieved"], "unit": entry["unit"], "ms_per_step": ms}

    vendor_line(args.workload, main_workload, args.steps)
    del main_workload["step"]

    others = {}
    if not args.only:
        # (the MFMA-only probe goes last: it heats the part more than any program does)
        for name, factory in sorted(workloads.items(), key=lambda item: item[0].startswith("mfma_ceiling")):
            if name == args.workload or name in ("copy_1gib", "mfma_ceiling_constant"):
                continue
            workload = factory()
            ms, wall = measure(workload, max(5, args.steps // 2), args.warmup)
            entry = roofline(workload, ms, traffic.get(name))
            entry["ms_per_step"] = ms
            # a step that the device finishes sooner than the host can ask for the next one (the 512^3 product)
            # is timed at the host's pace: the wall time says so, the single launches give the kernel's own time
            entry["wall_ms_per_step"] = wall
            entry["per_launch"] = per_launch(workload)
            entry["config"] = dict(workload["describe"], launch=launch_description(workload))
            others[name] = entry
            vendor_line(name, workload, max(5, args.steps // 2))
            del workload
            torch.cuda.empty_cache()

    result = {
        "metric": METRIC,
        "value": main_roofline["achieved"],
        "unit": main_roofline["unit"],
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": device_ms,
        "wall_ms_per_step": wall_ms,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16" if main_roofline["bound"] == "mfma" else "f32",
        "data": "synthetic" if args.inputs == "randn" else "synthetic, every operand a constant (diagnostic run: not the inputs the metric is quoted on)",
        "config": dict(main_workload["describe"], launch=launch_plan),
        "roofline": main_roofline,
        "per_launch": single,
        "l2": "not flushed between launches",
        "others": others,
        "vendor_gpu": vendor,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline_addmm()
        result["torch_cpu"] = torch_cpu_context()
        result["triton_interpreter_cpu"] = triton_interpreter_cpu()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
