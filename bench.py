#!/usr/bin/env python3
"""Benchmark of the JL projection hot path (and, beside it, the scoring GEMMs) on one MI355X.

`python bench.py [--gpus 1] [--steps K] [--warmup W]` prints ONE JSON line.

step      = one `trakhip_project` call on one resident batch [32, 11_689_512] fp16
            (ResNet-18-sized Rademacher projection to k = 4096, seed 7, 16 distinct batches
            cycled back to back; inputs are in HBM before the timed region starts).
value     = 2*B*P*k flop per step / time per step, in TFLOP/s.
roofline  = the projection kernel alone (phase 1 of the call), timed with HIP events recorded
            on the launch stream around every launch, against the dense fp16 MFMA peak.
cpu_baseline = the CPU restatement of trak's BasicProjector (oracle/basic_projector.py) timed on this host:
            the CPU-runnable configuration ([16, 1_048_576] fp32 -> 512) in full, the ResNet-9- and
            ResNet-18-sized configurations as two full 100-column blocks each, scaled by num_blocks / 2
            and flagged "extrapolated" (the BERT-sized one only with --cpu-c4).
sustained = the same calls back to back for --sustain seconds (default 2).
`scoring` = BasicScoreComputer at N=50_000, M=10_000, k=4096 fp32: GEMM TFLOP/s against the fp32
            MFMA peak, the SPD inverse separately, and a CPU sample beside it.
other_configs = whole calls (Python wrapper included) of the other benchmark configurations: c1 (fp32
            [16, 1_048_576] -> 512), c2 (ResNet-9-sized), c4 (BERT-sized chunked normal), the headline shape as
            a gradient dict, and projection dimensions 3072 and 15 360.
`--only NAME` runs one workload alone (for profiler runs): c1 | c2 | c3_b40 | c3_b48 | c3_b64 | c3_k1536 | c3_k3072 |
            c3_k15360 | c3_k40960 | c3_normal_b32 | c3_normal_b64 | c3_dict | c4 | c4_rademacher | vendor_gemm | scoring |
            general_inverse | mfma_rate.
"""
import argparse
import ctypes
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0   # MI355X dense fp16/bf16 MFMA
PEAK_FP32_TFLOPS = 157.3    # MI355X fp32 MFMA
# HBM bytes of one projection-kernel launch at the benchmark shape come from the tracked rocprofv3 summary
# (FETCH_SIZE and WRITE_SIZE in KiB per dispatch, each times the factor a 1 GiB copy needs for the same counter).
TRAFFIC_PROFILE = os.path.join("profiles", "jl_project_f16_rademacher_resnet18_hbm_counters.txt")


def profiled_kernel_traffic():
    """(bytes per launch, source file) read from the tracked HBM-counter summary, or (None, None)."""
    import re

    try:
        text = open(os.path.join(ROOT, TRAFFIC_PROFILE)).read()
        f = re.search(r"^\s*FETCH_SIZE\s+([\d.]+) KiB x ([\d.]+)", text, re.M)
        w = re.search(r"^\s*WRITE_SIZE\s+([\d.]+) KiB x ([\d.]+)", text, re.M)
        return (float(f.group(1)) * float(f.group(2)) + float(w.group(1)) * float(w.group(2))) * 1024, TRAFFIC_PROFILE
    except (OSError, AttributeError, ValueError):
        return None, None


METRIC = "JL proj TFLOP/s & % MFMA peak at P=11.7M,k=4096,B=32; scoring TFLOP/s"


class Hip:
    """Minimal HIP event API through ctypes (events on an explicit stream)."""

    def __init__(self):
        self.lib = ctypes.CDLL("libamdhip64.so")
        self.lib.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.lib.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        self.lib.hipEventSynchronize.argtypes = [ctypes.c_void_p]
        self.lib.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.lib.hipEventDestroy.argtypes = [ctypes.c_void_p]

    def event(self):
        e = ctypes.c_void_p()
        assert self.lib.hipEventCreate(ctypes.byref(e)) == 0
        return e

    def record(self, e, stream):
        assert self.lib.hipEventRecord(e, ctypes.c_void_p(stream)) == 0

    def elapsed_ms(self, a, b):
        assert self.lib.hipEventSynchronize(b) == 0
        ms = ctypes.c_float()
        assert self.lib.hipEventElapsedTime(ctypes.byref(ms), a, b) == 0
        return ms.value


def make_batches(torch, dev, n_batches, B, P, seed):
    """ResNet-18-sized synthetic gradients: 62 parameter blocks with log-uniform scales in
    [1e-5, 1e-2] times N(0,1), fp16, generated on the device."""
    gen = torch.Generator(device=dev).manual_seed(seed)
    blocks = 62
    edges = torch.linspace(0, P, blocks + 1).long().tolist()
    out = []
    for _ in range(n_batches):
        scale = 10 ** (torch.rand(blocks, generator=gen, device=dev) * 3 - 5)
        g = torch.empty(B, P, dtype=torch.float16, device=dev)
        for i in range(blocks):
            lo, hi = edges[i], edges[i + 1]
            g[:, lo:hi] = (torch.randn(B, hi - lo, generator=gen, device=dev) * scale[i]).half()
        out.append(g)
    return out


def bench_projection(torch, dev, steps, warmup, n_batches, sustain_s=2.0):
    from trak_amd import _lib, fast_jl

    lib = _lib.load()
    hip = Hip()
    B, P, k, seed = 32, 11_689_512, 4096, 7
    tiles = torch.cuda.get_device_properties(dev).multi_processor_count
    batches = make_batches(torch, dev, n_batches, B, P, 20_003)
    out = torch.empty(B, k, dtype=torch.float32, device=dev)
    ws = torch.empty(lib.trakhip_project_workspace(B, P, k, tiles), dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    vp = ctypes.c_void_p

    def full(g):
        _lib.check(lib.trakhip_project(vp(g.data_ptr()), _lib.F16, B, P, P, vp(out.data_ptr()), vp(ws.data_ptr()),
                                       ws.numel(), k, seed, tiles, _lib.RADEMACHER, vp(stream)))

    for i in range(warmup):
        full(batches[i % n_batches])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        full(batches[i % n_batches])
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / steps

    # the projection kernel alone: events around each phase-1 launch on the launch stream
    evs = [(hip.event(), hip.event()) for _ in range(steps)]
    for i in range(steps):
        g = batches[i % n_batches]
        hip.record(evs[i][0], stream)
        _lib.check(lib.trakhip_project_partials(vp(g.data_ptr()), _lib.F16, B, P, P, vp(ws.data_ptr()), ws.numel(), k,
                                                seed, tiles, _lib.RADEMACHER, vp(stream)))
        hip.record(evs[i][1], stream)
        _lib.check(lib.trakhip_project_reduce(vp(ws.data_ptr()), B, P, k, tiles, 1.0, vp(out.data_ptr()), vp(stream)))
    torch.cuda.synchronize()
    kernel_ms = sorted(hip.elapsed_ms(a, b) for a, b in evs)
    kernel_avg = sum(kernel_ms) / len(kernel_ms)
    flop = 2.0 * B * P * k

    # sustained: back-to-back calls over the resident batches for `sustain_s` seconds (the kernel's bound
    # is power, so a figure over seconds belongs beside the one over the timed steps)
    sustained = None
    if sustain_s > 0:
        n = max(steps, int(math.ceil(sustain_s * 1e3 / ms_per_step)))
        evs = [(hip.event(), hip.event()) for _ in range(n)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            g = batches[i % n_batches]
            hip.record(evs[i][0], stream)
            _lib.check(lib.trakhip_project_partials(vp(g.data_ptr()), _lib.F16, B, P, P, vp(ws.data_ptr()), ws.numel(),
                                                    k, seed, tiles, _lib.RADEMACHER, vp(stream)))
            hip.record(evs[i][1], stream)
            _lib.check(lib.trakhip_project_reduce(vp(ws.data_ptr()), B, P, k, tiles, 1.0, vp(out.data_ptr()), vp(stream)))
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        km = sorted(hip.elapsed_ms(a, b) for a, b in evs)
        sustained = {
            "calls": n, "seconds": round(wall, 3), "tflops": round(flop * n / wall / 1e12, 1),
            "kernel_ms_min": round(km[0], 4), "kernel_ms_median": round(km[n // 2], 4),
            "kernel_ms_max": round(km[-1], 4),
            "kernel_tflops_median": round(flop / km[n // 2] / 1e9, 1),
        }
    return {
        "sustained": sustained,
        "flop": flop,
        "ms_per_step": ms_per_step,
        "tflops": flop / (ms_per_step * 1e-3) / 1e12,
        "kernel_ms_avg": kernel_avg,
        "kernel_ms_min": kernel_ms[0],
        "kernel_tflops": flop / (kernel_avg * 1e-3) / 1e12,
        "tiles": tiles,
        "shape": {"B": B, "P": P, "k": k},
    }


def resnet18_param_shapes():
    """Parameter shapes of torchvision's resnet18 in `named_parameters()` order (62 tensors,
    11 689 512 elements)."""
    shapes = [(64, 3, 7, 7), (64,), (64,)]
    inp = 64
    for out, stride in ((64, 1), (128, 2), (256, 2), (512, 2)):
        for block in range(2):
            cin = inp if block == 0 else out
            shapes += [(out, cin, 3, 3), (out,), (out,), (out, out, 3, 3), (out,), (out,)]
            if block == 0 and (stride != 1 or inp != out):
                shapes += [(out, inp, 1, 1), (out,), (out,)]
        inp = out
    shapes += [(1000, 512), (1000,)]
    return shapes


def bench_featurize_path(torch, dev, reps=20):
    """The projector call of TRAKer.featurize on a ResNet-18 gradient dict: flatten-and-copy then
    project (what the reference does) against projecting the dict in place."""
    import math

    from trak_amd import CudaProjector, ProjectionType, vectorize

    shapes = resnet18_param_shapes()
    P = sum(math.prod(sh) for sh in shapes)
    assert P == 11_689_512 and len(shapes) == 62
    gen = torch.Generator(device=dev).manual_seed(20_006)
    grads = {i: (torch.randn(32, *sh, generator=gen, device=dev) * 1e-3).half() for i, sh in enumerate(shapes)}
    proj = CudaProjector(P, 4096, 7, ProjectionType.rademacher, dev, 32)

    def timed(fn):
        for _ in range(5):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / reps

    flat_ms = timed(lambda: proj.project(vectorize(grads, device=dev), 0))
    gather_ms = timed(lambda: proj.project(grads, 0))
    same = bool(torch.equal(proj.project(vectorize(grads, device=dev), 0), proj.project(grads, 0)))
    return {"vectorize_then_project_ms": flat_ms, "project_dict_in_place_ms": gather_ms, "bit_identical": same,
            "tflops_in_place": 2.0 * 32 * P * 4096 / gather_ms / 1e9}


def bench_batch_scaling(torch, dev):
    """Projection throughput against the number of gradient rows per call at the ResNet-18 shape."""
    from trak_amd import CudaProjector, ProjectionType

    P, k = 11_689_512, 4096
    proj = CudaProjector(P, k, 7, ProjectionType.rademacher, dev, 32)
    gen = torch.Generator(device=dev).manual_seed(20_007)
    res = {}
    for B in (32, 64, 128):
        g = (torch.randn(B, P, generator=gen, device=dev) * 1e-3).half()
        for _ in range(8):
            proj.project(g, 0)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(20):
            proj.project(g, 0)
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b) / 20
        res[f"B={B}"] = {"ms": ms, "ms_per_32_rows": ms * 32 / B, "tflops": 2.0 * B * P * k / ms / 1e9}
        del g
    return res


def _config_calls(torch, dev, name):
    """(call, flop per call, description) for one named projection configuration: the synthetic
    inputs of the benchmark configurations other than the headline one, resident on the device."""
    import numpy as np

    from trak_amd import ChunkedCudaProjector, CudaProjector, ProjectionType

    gen = torch.Generator(device=dev).manual_seed(20_001)
    if name == "c1":
        g = torch.randn(16, 1_048_576, generator=gen, device=dev) * 1e-3
        p = CudaProjector(1_048_576, 512, 42, ProjectionType.rademacher, dev, 32)
        return (lambda: p.project(g, 0)), 2.0 * 16 * 1_048_576 * 512, "fp32 rademacher [16,1048576] -> 512"
    if name == "c2":
        g = (torch.randn(32, 4_825_610, generator=gen, device=dev) * 5e-4).half()
        g[torch.rand(32, 4_825_610, generator=gen, device=dev) < 0.01] = 0
        p = CudaProjector(4_825_610, 2048, 0, ProjectionType.rademacher, dev, 32)
        return (lambda: p.project(g, 0)), 2.0 * 32 * 4_825_610 * 2048, "fp16 rademacher [32,4825610] -> 2048"
    if name == "c3_b64":
        P = sum(math.prod(sh) for sh in resnet18_param_shapes())
        g = (torch.randn(64, P, generator=gen, device=dev) * 1e-3).half()
        p = CudaProjector(P, 4096, 7, ProjectionType.rademacher, dev, 32)
        return (lambda: p.project(g, 0)), 2.0 * 64 * P * 4096, "fp16 rademacher [64,11689512] -> 4096 (one pass of 64 rows)"
    if name in ("c3_k1536", "c3_k3072", "c3_k15360", "c3_k40960", "c3_b40", "c3_b48"):
        # the benchmark shape at other projection dimensions (the reference's tests use 15 360, its
        # documentation recommends 1 000 - 40 000) and at batch sizes between one and two 32-row blocks
        P = sum(math.prod(sh) for sh in resnet18_param_shapes())
        k = int(name[4:]) if name[3] == "k" else 4096
        B = int(name[4:]) if name[3] == "b" else 32
        g = (torch.randn(B, P, generator=gen, device=dev) * 1e-3).half()
        p = CudaProjector(P, k, 7, ProjectionType.rademacher, dev, 32)
        return (lambda: p.project(g, 0)), 2.0 * B * P * k, f"fp16 rademacher [{B},{P}] -> {k}"
    if name in ("c3_normal_b32", "c3_normal_b64"):
        B = int(name[-2:])
        P = sum(math.prod(sh) for sh in resnet18_param_shapes())
        g = (torch.randn(B, P, generator=gen, device=dev) * 1e-3).bfloat16()
        p = CudaProjector(P, 4096, 7, ProjectionType.normal, dev, 32)
        return (lambda: p.project(g, 0)), 2.0 * B * P * 4096, f"bf16 normal [{B},11689512] -> 4096 (one pass)"
    if name == "c3_dict":
        shapes = resnet18_param_shapes()
        P = sum(math.prod(sh) for sh in shapes)
        grads = {i: (torch.randn(32, *sh, generator=gen, device=dev) * 1e-3).half() for i, sh in enumerate(shapes)}
        p = CudaProjector(P, 4096, 7, ProjectionType.rademacher, dev, 32)
        return (lambda: p.project(grads, 0)), 2.0 * 32 * P * 4096, "fp16 rademacher ResNet-18 gradient dict (62 tensors) -> 4096"
    if name in ("c4", "c4_rademacher"):
        chunk = 27_370_560
        seeds = np.random.default_rng(123).integers(0, 500, size=4)
        pt = ProjectionType.normal if name == "c4" else ProjectionType.rademacher
        # Student-t (nu = 3) scaled by 1e-4: normal / sqrt(chi2_3 / 3)
        grads = {}
        for i in range(4):
            z = torch.randn(32, chunk, generator=gen, device=dev)
            c = torch.randn(3, 32, chunk, generator=gen, device=dev, dtype=torch.float16).float().square_().sum(0)
            grads[i] = (z * torch.rsqrt(c / 3.0) * 1e-4).bfloat16()
            del z, c
        per = [CudaProjector(chunk, 4096, int(seeds[i]), pt, dev, 32) for i in range(4)]
        p = ChunkedCudaProjector(per, chunk, [chunk] * 4, 32, dev, torch.bfloat16)
        return (lambda: p.project(grads, 0)), 2.0 * 32 * 4 * chunk * 4096, \
            f"bf16 {pt.value} chunked (4 x 27370560) [32,109482240] -> 4096"
    raise ValueError(f"unknown configuration {name}")


def bench_config(torch, dev, name, reps, warm_seconds=0.1, min_seconds=0.25):
    """Whole calls back to back: at least `warm_seconds` of untimed calls first (the clocks of an idle GPU take
    tens of milliseconds to come up), then at least `reps` calls and `min_seconds` between two events."""
    call, flop, what = _config_calls(torch, dev, name)
    call()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    call()
    torch.cuda.synchronize()
    one = max(time.perf_counter() - t0, 1e-5)
    for _ in range(min(2000, int(warm_seconds / one))):
        call()
    reps = max(reps, min(5000, int(min_seconds / one)))
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        call()
    b.record()
    torch.cuda.synchronize()
    ms = a.elapsed_time(b) / reps
    return {"what": what, "ms": ms, "tflops": flop / ms / 1e9, "calls": reps}


def bench_general_inverse(torch, dev, n=4096, reps=3):
    """The inverse of a Gram matrix that is not positive definite (rounded to fp16) at proj_dim n: this library's
    pivoted elimination against the Cholesky route on the same matrix plus a ridge, and torch.linalg.inv (the
    reference's call, the vendor's LU) for comparison."""
    from trak_amd.utils import general_inverse, spd_inverse

    gen = torch.Generator(device=dev).manual_seed(5)
    q, _ = torch.linalg.qr(torch.randn(n, n, generator=gen, device=dev, dtype=torch.float64))
    spectrum = 1000.0 / torch.arange(1, n + 1, dtype=torch.float64, device=dev) ** 1.5
    gram = ((q * spectrum) @ q.T).half().float()
    del q

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / reps

    return {"n": n, "general_inverse_ms": timed(lambda: general_inverse(gram, normalize=True)),
            "spd_inverse_with_ridge_ms": timed(lambda: spd_inverse(gram, lambda_reg=1.0, normalize=True)),
            "torch_linalg_inv_ms": timed(lambda: torch.linalg.inv(gram))}


MFMA_RATE_CASES = [
    # name, instruction (0 f16, 1 bf16, 2 f32), operand kind of A, of B (see trak_amd/csrc/mfma_rate.hip)
    ("f16 A=0 B=0", 0, 0, 0),
    ("f16 A=gradient-like B=+-1 (as the projection kernel)", 0, 1, 2),
    ("f16 A=+-1 B=gradient-like (swapped)", 0, 2, 1),
    ("f16 A=random B=random", 0, 3, 3),
    ("bf16 A=random B=random (as the 16-bit GEMM kernels)", 1, 4, 4),
    ("f32 A=random B=random (v_mfma_f32_32x32x2_f32)", 2, 3, 3),
]


def bench_vendor_gemm(torch, dev, reps=6):
    """The scores product of the fp16 scoring section through torch.mm (hipBLASLt), fp32 result: the
    library kernel that `gemm_nt16_kernel` is compared with, on the same operands, for profiler runs."""
    g = torch.Generator(device=dev).manual_seed(1)
    out = {}
    for name, dt in (("fp16", torch.float16), ("bf16", torch.bfloat16)):
        X = (torch.randn(50_000, 4096, generator=g, device=dev) / 64).to(dt)
        T = (torch.randn(10_000, 4096, generator=g, device=dev) / 64).to(dt)
        for _ in range(3):
            torch.mm(X, T.T, out_dtype=torch.float32)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            torch.mm(X, T.T, out_dtype=torch.float32)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) / reps * 1e3
        out[name] = {"scores_ms": ms, "tflops": 2.0 * 50_000 * 10_000 * 4096 / (ms * 1e-3) / 1e12}
        del X, T
    return out


def bench_mfma_rate(torch, dev, iters=300_000):
    """What a loop of nothing but independent MFMAs sustains on this machine, by operand data (the
    clock is power limited, so the rate depends on the data): the reference point for the projection
    and GEMM kernels.  One dispatch per case, timed with events on the launch stream."""
    path = os.path.join(ROOT, "trak_amd", "libtrakhip_diag.so")
    if not os.path.exists(path):  # not part of the product build: made when this workload asks for it
        from trak_amd.build import build_diag

        build_diag(verbose=False)
    lib = ctypes.CDLL(path)
    lib.trakhip_diag_mfma_rate_out_floats.restype = ctypes.c_size_t
    lib.trakhip_diag_mfma_rate.restype = ctypes.c_double
    lib.trakhip_diag_mfma_rate.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p, ctypes.c_void_p]
    out = torch.empty(lib.trakhip_diag_mfma_rate_out_floats(), dtype=torch.float32, device=dev)
    stream = torch.cuda.current_stream(dev).cuda_stream
    res = {}
    for name, instr, ka, kb in MFMA_RATE_CASES:
        lib.trakhip_diag_mfma_rate(instr, ka, kb, 20_000, out.data_ptr(), stream)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        flop = lib.trakhip_diag_mfma_rate(instr, ka, kb, iters, out.data_ptr(), stream)
        b.record()
        torch.cuda.synchronize()
        assert flop > 0
        ms = a.elapsed_time(b)
        res[name] = {"ms": round(ms, 2), "tflops": round(flop / ms / 1e9, 1)}
    return res


OTHER_CONFIGS = (
    # name, timed calls, what bounds the kernel (the peak its TFLOP/s is a fraction of)
    ("c1", 200, "bf16 MFMA (fp32 gradients split exactly into three bf16 terms: three MFMAs per step)"),
    ("c2", 100, "fp16 MFMA"),
    ("c3_dict", 10, "fp16 MFMA"),
    ("c3_k3072", 10, "fp16 MFMA"),
    ("c3_k15360", 6, "fp16 MFMA"),
    ("c4", 3, "vector ALU (a normal entry costs about 8 issue slots and is used for 32 multiply-adds); "
              "fraction of the fp16 MFMA peak given for comparison"),
)


def bench_other_configs(torch, dev, names=None):
    """Whole-call throughput (Python wrapper included) of the other benchmark configurations - the
    CPU-runnable fp32 case, the ResNet-9-sized case, the BERT-sized chunked normal case -, of the
    headline shape given as a gradient dict, and of projection dimensions whose column-block count
    does not divide the CU count."""
    res = {}
    for name, reps, bound in OTHER_CONFIGS:
        if names is not None and name not in names:
            continue
        r = bench_config(torch, dev, name, reps)
        res[name] = {"what": r["what"], "ms": round(r["ms"], 4), "tflops": round(r["tflops"], 1),
                     "frac_fp16_mfma_peak": round(r["tflops"] / PEAK_FP16_TFLOPS, 4), "bound": bound, "calls": r["calls"]}
        torch.cuda.empty_cache()
    return res


def bench_store_paths(torch, dev):
    """The store-side epilogues against the reference's sequences of passes: one featurize batch at
    the ResNet-18 shape down to host memory (trak/traker.py:425-429), and the score sums of three
    checkpoints at N=50 000, M=10 000 down to a host array (trak/traker.py:641-678)."""
    import numpy as np

    from trak_amd import BasicScoreComputer, CudaProjector, FeatureWriter, ProjectionType, ScoreAccumulator

    res = {}
    P, k, B = 11_689_512, 4096, 32
    proj = CudaProjector(P, k, 7, ProjectionType.rademacher, dev, 32)
    gen = torch.Generator(device=dev).manual_seed(20_008)
    g = (torch.randn(B, P, generator=gen, device=dev) * 1e-3).half()
    nf = torch.sqrt(torch.tensor(float(P)))
    store = np.zeros((64 * B, k), dtype=np.float16)

    def reference_batch(i):
        x = proj.project(g, 0)
        x /= nf
        store[i * B:(i + 1) * B] = x.to(torch.float16).cpu().clone().detach().numpy()

    writer = FeatureWriter(proj, k, nf, dtype=torch.float16, max_batch_size=B, depth=2)

    def fused_batch(i):
        writer.write(g, 0, store, np.arange(i * B, (i + 1) * B))

    for name, fn, done in (("reference_sequence", reference_batch, lambda: None),
                           ("feature_writer", fused_batch, writer.flush)):
        for i in range(4):
            fn(i)
        done()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(64):
            fn(i)
        done()
        torch.cuda.synchronize()
        res[f"featurize_batch_to_host_ms[{name}]"] = (time.perf_counter() - t0) * 1e3 / 64
    del g

    N, M, kk, models = 50_000, 10_000, 4096, 3
    sc = BasicScoreComputer(dtype=torch.float32, device=dev)
    f = torch.randn(N, kk, generator=gen, device=dev) / 64
    t = torch.randn(M, kk, generator=gen, device=dev) / 64
    o = np.random.default_rng(0).random((N, 1)).astype(np.float32)
    out = np.zeros((N, M), dtype=np.float32)
    for _ in range(2):  # second pass timed: the first touches the host pages
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        acc = torch.zeros(N, M)
        osum = np.zeros((N, 1), dtype=np.float32)
        for _m in range(models):
            sc.get_scores(f, t, accumulator=acc)
            osum += o
        out[:] = (acc.numpy() / float(models)) * (osum / float(models))
        ref_s = time.perf_counter() - t0
    del acc
    for _ in range(2):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        sa = ScoreAccumulator(sc, N, M)
        for _m in range(models):
            sa.add(f, t, o)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        sa.finalize(out)
        t2 = time.perf_counter()
        del sa
    res["finalize_scores_3_checkpoints_s[reference_sequence]"] = ref_s
    res["finalize_scores_3_checkpoints_s[score_accumulator]"] = t2 - t0
    res["score_accumulator_finalize_only_s"] = t2 - t1
    res["score_accumulator_finalize_GBps"] = N * M * 4 / (t2 - t1) / 1e9
    return res


def bench_scoring(torch, dev, reps=3):
    from trak_amd import BasicScoreComputer

    N, M, k, lam = 50_000, 10_000, 4096, 1e-3
    gen = torch.Generator(device=dev).manual_seed(20_005)
    X = torch.randn(N, k, generator=gen, device=dev) / 64
    Xt = torch.randn(M, k, generator=gen, device=dev) / 64
    otl = torch.rand(N, generator=gen, device=dev)
    sc = BasicScoreComputer(dtype=torch.float32, device=dev, lambda_reg=lam)

    def timed(fn):
        best = None
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            r = fn()
            b.record()
            torch.cuda.synchronize()
            ms = a.elapsed_time(b)
            best = ms if best is None else min(best, ms)
        return r, best

    from trak_amd.utils import gemm_nt, gemm_nt16, gemm_nt_split, gemm_tn, gram_split, spd_inverse, split2_rows, split_rows

    # the fp32 MFMA instruction (v_mfma_f32_32x32x2_f32): priced against the 157.3 TFLOP/s fp32 peak
    xtx, t_xtx = timed(lambda: gemm_tn(X, X))
    (inv, _), t_inv = timed(lambda: spd_inverse(xtx, lambda_reg=lam, normalize=True))
    feats, t_feat = timed(lambda: gemm_nt(X, inv))
    scores, t_sc = timed(lambda: gemm_nt(feats, Xt, row_scale=otl))
    gemm_flop = 2.0 * N * k * k * 2 + 2.0 * N * M * k
    gemm_ms = t_xtx + t_feat + t_sc
    del scores
    # the same three products with fp32 operands split exactly into three bf16 terms (six bf16 MFMAs
    # per k step, fp32 accumulation; what BasicScoreComputer runs by default), splitting included:
    # fp32-equivalent TFLOP/s = the same 2*M*N*K over the time; 6x that many bf16 flops are executed
    _, s_xtx = timed(lambda: gram_split(split_rows(X, transposed=True)))  # lower-triangle tiles + mirror
    _, s_feat = timed(lambda: gemm_nt_split(split_rows(X), split_rows(inv)))
    _, s_sc = timed(lambda: gemm_nt_split(split_rows(feats), split_rows(Xt), row_scale=otl))
    split_ms = s_xtx + s_feat + s_sc
    # opt-in cheaper split (BasicScoreComputer(gemm="split2")): rows scaled by powers of two, two fp16
    # planes, three fp16 MFMAs per k step; entries keep 22 significand bits relative to their row's maximum
    _, q_xtx = timed(lambda: gram_split(split2_rows(X, transposed=True)))
    _, q_feat = timed(lambda: gemm_nt_split(split2_rows(X), split2_rows(inv)))
    _, q_sc = timed(lambda: gemm_nt_split(split2_rows(feats), split2_rows(Xt), row_scale=otl))
    split2_ms = q_xtx + q_feat + q_sc
    # TRAKer's default stores gradients and features as fp16 (use_half_precision): the same products
    # with one MFMA per k step and exact products; X^T X from one fp16 plane (the transposed operand
    # needs the re-layout), the two row-major products read in place (what BasicScoreComputer runs)
    Xh, invh, fh, Xth = X.half(), inv.half(), feats.half(), Xt.half()
    _, h_xtx = timed(lambda: gram_split(split_rows(Xh, transposed=True)))
    _, h_feat = timed(lambda: gemm_nt16(Xh, invh))
    _, h_sc = timed(lambda: gemm_nt16(fh, Xth, row_scale=otl))
    del Xh, fh, Xth
    # X^T X is computed on the tiles that touch the lower triangle only (256 x 256 tiles) and mirrored:
    # its flops are counted as computed, not as 2*N*k*k
    t256 = (k + 255) // 256
    split_flop = 2.0 * N * k * k * (1.0 + t256 * (t256 + 1) / 2.0 / (t256 * t256)) + 2.0 * N * M * k
    return {
        "shape": {"N": N, "M": M, "k": k, "lambda": lam},
        "xtx_ms": t_xtx, "inverse_ms": t_inv, "x_xtx_inv_ms": t_feat, "scores_ms": t_sc,
        "gemm_tflops": gemm_flop / (gemm_ms * 1e-3) / 1e12,
        "gemm_frac_fp32_mfma_peak": gemm_flop / (gemm_ms * 1e-3) / 1e12 / PEAK_FP32_TFLOPS,
        "split_bf16x3": {
            "xtx_ms": s_xtx, "x_xtx_inv_ms": s_feat, "scores_ms": s_sc,
            "gemm_tflops_algorithmic": gemm_flop / (split_ms * 1e-3) / 1e12,  # 4*N*k*k + 2*N*M*k over the time
            "gemm_tflops_fp32_equivalent": split_flop / (split_ms * 1e-3) / 1e12,
            "frac_fp32_mfma_peak": split_flop / (split_ms * 1e-3) / 1e12 / PEAK_FP32_TFLOPS,
            "bf16_mfma_tflops_executed": 6 * split_flop / (split_ms * 1e-3) / 1e12,
            "frac_bf16_mfma_peak": 6 * split_flop / (split_ms * 1e-3) / 1e12 / PEAK_FP16_TFLOPS,
            "xtx_note": "symmetric product: lower-triangle tiles computed and mirrored, flops counted as computed",
        },
        "split_fp16x2_opt_in": {
            "xtx_ms": q_xtx, "x_xtx_inv_ms": q_feat, "scores_ms": q_sc,
            "gemm_tflops_algorithmic": gemm_flop / (split2_ms * 1e-3) / 1e12,
            "gemm_tflops_fp32_equivalent": split_flop / (split2_ms * 1e-3) / 1e12,
            "note": "not the default: operand error up to 2^-22 relative to the row maximum (three-plane split: exact)",
        },
        "fp16_inputs": {
            "xtx_ms": h_xtx, "x_xtx_inv_ms": h_feat, "scores_ms": h_sc,
            "gemm_tflops": split_flop / ((h_xtx + h_feat + h_sc) * 1e-3) / 1e12,
            "frac_fp16_mfma_peak": split_flop / ((h_xtx + h_feat + h_sc) * 1e-3) / 1e12 / PEAK_FP16_TFLOPS,
        },
        "inverse_flop": float(k) ** 3,
        "scores_orientation": "[N_train, M_targets]",
    }


def cpu_baseline(torch, cpu_c4=False):
    """trak's BasicProjector CPU path (restated in oracle/basic_projector.py) on its CPU-runnable
    configuration, all host cores; plus a bounded BasicScoreComputer sample."""
    from oracle.basic_projector import BasicProjectorCPU
    from oracle.score_oracle import BasicScoreComputerCPU

    cores = int(os.environ.get("OMP_NUM_THREADS", 0)) or os.cpu_count()
    torch.set_num_threads(cores)
    B, P, k = 16, 1_048_576, 512
    gen = torch.Generator().manual_seed(20_001)
    g = torch.randn(B, P, generator=gen) * 1e-3
    proj = BasicProjectorCPU(grad_dim=P, proj_dim=k, seed=42, proj_type="rademacher")
    t0 = time.perf_counter()
    proj.project(g, model_id=0)
    dt = time.perf_counter() - t0
    flop = 2.0 * B * P * k
    res = {
        "value": flop / dt / 1e12, "unit": "TFLOP/s", "cores": cores, "kind": "port",
        "sample": f"BasicProjector restatement, full config [16,1048576] fp32 -> 512 rademacher, {dt:.2f} s",
    }
    # The larger projection configurations take minutes to hours on a CPU (every 100-column block regenerates
    # a [P, 100] fp32 matrix): two full blocks are timed and the time is scaled by num_blocks / 2
    # (trak/projectors.py:258-314 does the same work for every block).  fp32, as BasicProjector runs on a CPU.
    def sample(B, P, k, seed, proj_type, scale, chunks=1):
        g = torch.randn(B, P, generator=gen) * scale
        pr = BasicProjectorCPU(grad_dim=P, proj_dim=k, seed=seed, proj_type=proj_type)
        blocks = 2
        t0 = time.perf_counter()
        pr.project(g, model_id=0, max_blocks=blocks)
        dt = time.perf_counter() - t0
        full = dt * pr.num_blocks / blocks * chunks
        return {"tflops": 2.0 * B * P * chunks * k / full / 1e12, "extrapolated": True, "blocks_timed": blocks,
                "blocks_total": pr.num_blocks * chunks, "sample_s": round(dt, 2), "estimated_full_s": round(full, 1)}

    res["other_configs"] = {
        "c2_[32,4825610]_k2048_rademacher": sample(32, 4_825_610, 2048, 0, "rademacher", 5e-4),
        "c3_[32,11689512]_k4096_rademacher": sample(32, 11_689_512, 4096, 7, "rademacher", 1e-3),
    }
    if cpu_c4:
        # one of the four parameter chunks; the other three cost the same
        res["other_configs"]["c4_[32,109482240]_k4096_normal_4_chunks"] = sample(32, 27_370_560, 4096, 123, "normal",
                                                                                 1e-4, chunks=4)
    N, M, kk = 50_000, 10_000, 4096  # the scoring configuration in full
    X = torch.randn(N, kk, generator=gen) / 64
    Xt = torch.randn(M, kk, generator=gen) / 64
    sc = BasicScoreComputerCPU(lambda_reg=1e-3)
    t0 = time.perf_counter()
    xtx = sc.get_xtx(X)
    f = sc.get_x_xtx_inv(X, xtx)
    acc = torch.zeros(N, M)
    sc.get_scores(f, Xt, acc)
    dts = time.perf_counter() - t0
    res["scoring_tflops"] = (4.0 * N * kk * kk + 2.0 * N * M * kk) / dts / 1e12
    res["scoring_sample"] = f"BasicScoreComputer restatement N={N}, M={M}, k={kk} fp32, {dts:.2f} s (inverse included)"
    try:
        with open("/proc/cpuinfo") as f:
            res["cpu_model"] = next(l.split(":", 1)[1].strip() for l in f if l.startswith("model name"))
    except (OSError, StopIteration):
        res["cpu_model"] = "unknown"
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--batches", type=int, default=16, help="distinct resident batches cycled through")
    ap.add_argument("--sustain", type=float, default=2.0,
                    help="seconds of back-to-back calls for the `sustained` figure (0 = skip)")
    ap.add_argument("--cpu-c4", action="store_true",
                    help="also time the BERT-sized normal configuration's BasicProjector sample on the CPU (about a minute)")
    ap.add_argument("--no-scoring", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-other-configs", action="store_true",
                    help="skip the other projection configurations (`other_configs` of the JSON line)")
    ap.add_argument("--all-configs", action="store_true",
                    help="also time the featurize / store paths and batch scaling and print them to stderr")
    ap.add_argument("--only", default=None, metavar="NAME",
                    help="run just one workload for --steps calls and print its timing (for profiler runs): "
                         "c1 | c2 | c3_b40 | c3_b48 | c3_b64 | c3_k1536 | c3_k3072 | c3_k15360 | c3_k40960 | c3_normal_b32 | "
                         "c3_normal_b64 | c3_dict | c4 | c4_rademacher | scoring | general_inverse | mfma_rate | vendor_gemm "
                         "(torch.mm on the scoring operands, for comparison)")
    ap.add_argument("--steady", action="store_true",
                    help="with --only: at least 0.1 s of untimed calls first and at least 0.25 s timed (for timing without "
                         "a profiler: an idle GPU's clocks take tens of milliseconds to come up)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 1 GiB device-to-device copy (reference point for rocprofv3 byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this library has no multi-GPU path (the projection shards over rows, "
              "columns or parameters without changing the kernel); run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    if args.copy_calibration:
        src = torch.ones(1 << 29, dtype=torch.float16, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    if args.only:
        if args.only == "mfma_rate":
            print(json.dumps({"only": "mfma_rate", **bench_mfma_rate(torch, dev)}))
        elif args.only == "vendor_gemm":
            print(json.dumps({"only": "vendor_gemm", **bench_vendor_gemm(torch, dev)}))
        elif args.only == "general_inverse":
            print(json.dumps({"only": "general_inverse", **bench_general_inverse(torch, dev)}))
        elif args.only == "scoring":
            print(json.dumps({"only": "scoring", **bench_scoring(torch, dev, reps=max(1, min(args.steps, 3)))}))
        else:
            # exactly --steps calls after one warm-up call (profiler runs); --steady: warmed up and timed by wall time
            w, m = (0.1, 0.25) if args.steady else (0.0, 0.0)
            print(json.dumps({"only": args.only, **bench_config(torch, dev, args.only, args.steps, w, m)}))
        return
    proj = bench_projection(torch, dev, args.steps, args.warmup, args.batches, args.sustain)
    torch.cuda.empty_cache()
    other = None if args.no_other_configs else bench_other_configs(torch, dev)
    if args.all_configs:
        print(json.dumps(bench_config(torch, dev, "c4_rademacher", 5), indent=1), file=sys.stderr)
        print(json.dumps({"featurize_path": bench_featurize_path(torch, dev)}, indent=1), file=sys.stderr)
        print(json.dumps({"batch_scaling": bench_batch_scaling(torch, dev)}, indent=1), file=sys.stderr)
        torch.cuda.empty_cache()
        print(json.dumps({"store_paths": bench_store_paths(torch, dev)}, indent=1), file=sys.stderr)
        torch.cuda.empty_cache()
    scoring = None if args.no_scoring else bench_scoring(torch, dev)
    torch.cuda.empty_cache()
    cpu = None if args.no_cpu else cpu_baseline(torch, args.cpu_c4)

    traffic, traffic_source = profiled_kernel_traffic()
    line = {
        "metric": METRIC,
        "value": round(proj["tflops"], 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(proj["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {
            "workload": "ResNet-18-sized Rademacher JL projection: gradients [32, 11689512] fp16 "
                        "(62 blocks, log-uniform scales 1e-5..1e-2), k=4096, seed 7, "
                        f"{args.batches} resident batches cycled, num_feature_tiles={proj['tiles']}",
            "flop_per_step": proj["flop"],
            "frac_fp16_mfma_peak": round(proj["tflops"] / PEAK_FP16_TFLOPS, 4),
        },
        "roofline": {
            "bound": "mfma",
            "achieved": round(proj["kernel_tflops"], 3),
            "peak": PEAK_FP16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(proj["kernel_tflops"] / PEAK_FP16_TFLOPS, 4),
            "traffic": traffic,
            "traffic_unit": "bytes per launch (algorithmic input+output: %d)" % (32 * 11_689_512 * 2 + 32 * 4096 * 4),
            "traffic_source": traffic_source,
            "kernel": "jl_project_kernel<f16, rademacher>",
            "kernel_ms_avg": round(proj["kernel_ms_avg"], 4),
            "kernel_ms_min": round(proj["kernel_ms_min"], 4),
        },
        "sustained": proj["sustained"],
        "other_configs": other,
        "cpu_baseline": cpu,
        "scoring": scoring,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
