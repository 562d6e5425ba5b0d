#!/usr/bin/env python3
"""Attention hot-path benchmark on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3] [--report]

A step is one pass of the hot path over one batch of synthetic input: forward, then the
backward pre-pass (delta), dK/dV and dQ, called through the C ABI on tensors that are already
resident in HBM. The default workload is C3 (bf16, causal, B=2 H=16 S=4096 D=128), the one the
headline metric is quoted on. Rank 0 prints ONE JSON line on stdout; --report additionally
prints forward and forward+backward figures for all five configurations on stderr.

Order of a run: the CPU baselines first (the GPU idles meanwhile), then the per-configuration and
sibling-operation figures, and the headline region (W warm-up steps, K timed steps) LAST, directly
after them. An MI355X that has idled takes some tens of milliseconds of load to raise its clocks: timed
right after start-up, 5 warm-up steps (3 ms) are not enough and the same K steps take about 12 % longer
(that figure is reported as `cold_start`). `value` is the sustained rate.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"bf16": 2516.6, "fp16": 2516.6, "fp32": 157.3}  # MI355X dense MFMA peaks (256 CU x 2.4 GHz)
HBM_PEAK_GBS = 8000.0



def measured_traffic(workload, kernel):
    """HBM bytes (read + written) per launch of a kernel as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE:
    parsed from the summary profiles/<workload>_hbm_traffic.txt (columns: kernel, FETCH_SIZE KiB, scaled read MiB,
    WRITE_SIZE KiB, written MiB); None where no summary covers the kernel."""
    path = os.path.join(ROOT, "profiles", f"{workload.lower()}_hbm_traffic.txt")
    if not os.path.exists(path):
        return None
    for line in open(path):
        if not line.startswith("# " + kernel + " "):
            continue
        nums = []
        for tok in line.split():
            try:
                nums.append(float(tok))
            except ValueError:
                pass
        if len(nums) >= 4:
            return int((nums[1] + nums[3]) * 2**20)
    return None


def _dtype_name(dtype):
    import torch

    return {torch.float32: "fp32", torch.float16: "fp16", torch.bfloat16: "bf16"}[dtype]


class Path:
    """The four C-ABI calls of one step on preallocated device tensors."""

    def __init__(self, w, dev):
        import torch

        from trident_amd import _lib, operation, workloads

        self.w = w
        self.lib = _lib.lib()
        self.check = _lib.check
        q, k, v, d_o, mask = workloads.make_inputs(w)
        self.q, self.k, self.v, self.d_o = [x.to(dev) for x in (q, k, v, d_o)]
        self.mask = None if mask is None else mask.to(dev)
        B, H, S, D = self.q.shape
        self.o = torch.empty_like(self.q)
        self.lse = torch.empty(B, H, S, device=dev, dtype=torch.float32)
        self.delta = torch.empty_like(self.lse)
        self.dq, self.dk, self.dv = [torch.empty_like(self.q) for _ in range(3)]
        mview = operation._expand_mask(self.mask, (B, H, S, S)) if self.mask is not None else None
        self.mview = mview
        args = operation._make_args(self.q, self.k, self.v, self.o, self.lse, mview, w.dropout_p, w.is_causal, w.scale,
                                    w.dropout_seed, 0, self.d_o, self.dq, self.dk, self.dv, None, self.delta)
        self.args = args
        ref = ctypes.byref(args)
        # A step is the launch sequence of the operator (tri_attn_fwd, then what tri_attn_bwd launches): where
        # the fused dQ + delta kernel applies, dQ (with delta) and dK/dV; otherwise delta, dK/dV, dQ.
        self.kernels = []
        if mview is not None and self.lib.tri_attn_mask_classes_size(ref) > 0:
            # the classification of the mask's blocks is part of the step (a caller that reuses a mask pays it once)
            self.classes = torch.empty(self.lib.tri_attn_mask_classes_size(ref), dtype=torch.uint8, device=dev)
            args.mask_classes = self.classes.data_ptr()
            self.kernels.append(("mask_classes", lambda: self.check(self.lib.tri_attn_classify_mask(ref))))
            self.check(self.lib.tri_attn_classify_mask(ref))
        self.kernels.append(("fwd", lambda: self.check(self.lib.tri_attn_fwd(ref))))
        if w.backward:
            self.check(self.lib.tri_attn_fwd(ref))
            rc = self.lib.tri_attn_bwd_dq_delta(ref)
            if rc == 0:
                self.kernels += [
                    ("bwd_dq", lambda: self.check(self.lib.tri_attn_bwd_dq_delta(ref))),
                    ("bwd_dkdv", lambda: self.check(self.lib.tri_attn_bwd_dkdv(ref))),
                ]
            elif rc == _lib.ENOFUSE:
                self.kernels += [
                    ("bwd_delta", lambda: self.check(self.lib.tri_attn_bwd_delta(ref))),
                    ("bwd_dkdv", lambda: self.check(self.lib.tri_attn_bwd_dkdv(ref))),
                    ("bwd_dq", lambda: self.check(self.lib.tri_attn_bwd_dq(ref))),
                ]
            else:
                self.check(rc)

    def algorithmic_flops(self, kernel):
        """Flops credited per launch: forward 4 B H S^2 D; of the 10 B H S^2 D of the backward,
        dK/dV is credited its four GEMMs (S, dP, dV, dK) and dQ one (dQ); the S and dP that the
        dQ pass recomputes are not credited. Causal halves everything."""
        unit = self.w.flops() / 4.0  # 1 * B H S^2 D (x 1/2 causal)
        return {"fwd": 4.0, "bwd_dkdv": 8.0, "bwd_dq": 2.0, "bwd_delta": 0.0, "mask_classes": 0.0}[kernel] * unit

    def algorithmic_bytes(self, kernel):
        B, H, S, D = self.q.shape
        elt = self.q.element_size()
        if kernel == "bwd_delta":
            return 2 * B * H * S * D * elt + 4 * B * H * S
        return None


def run_steps(path, steps, warmup):
    """Returns (ms per step by wall clock, {kernel: avg ms} from HIP events on the launch stream).

    Every timed step brackets ONE of its kernels with a pair of events, step s the kernel s mod n: an event record is
    a packet of its own in the queue, and a pair around every kernel of every step makes the step 2-3 % longer than
    the same launches back to back. A kernel's average is over the steps that bracketed it."""
    import torch

    for _ in range(warmup):
        for _, fn in path.kernels:
            fn()
    torch.cuda.synchronize()
    n = len(path.kernels)
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(steps):
        for i, (_, fn) in enumerate(path.kernels):
            if i == s % n:
                events[s][0].record()
                fn()
                events[s][1].record()
            else:
                fn()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    per_kernel = {}
    for i, (name, fn) in enumerate(path.kernels):
        samples = [events[s][0].elapsed_time(events[s][1]) for s in range(steps) if s % n == i]
        if not samples:  # fewer steps than kernels: one more launch of this kernel, outside the timed region
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            samples = [e0.elapsed_time(e1)]
        per_kernel[name] = sum(samples) / len(samples)
    return wall_ms, per_kernel


def operator_ms(w, dev, steps, warmup):
    """The same step through the operator API (trident_amd.function + autograd): what a user of the
    reference's interface sees, including output allocation and the Python wrapper."""
    import torch

    import trident_amd
    from trident_amd import workloads

    q, k, v, d_o, mask = workloads.make_inputs(w)
    q, k, v, d_o = [x.to(dev) for x in (q, k, v, d_o)]
    mask = None if mask is None else mask.to(dev)
    if w.dropout_p:
        trident_amd.config.dropout_seed = (w.dropout_seed, 0)
    for x in (q, k, v):
        x.requires_grad_(w.backward)

    def step():
        out = trident_amd.function.scaled_dot_product_attention(q, k, v, attn_mask=mask, dropout_p=w.dropout_p,
                                                                is_causal=w.is_causal)
        if w.backward:
            out.backward(d_o)
            q.grad = k.grad = v.grad = None

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def cpu_baseline(w, reps=3):
    """torch.nn.functional.scaled_dot_product_attention on the host cores (the op the reference's
    tests take as their oracle), forward (+ backward) on the same workload."""
    import torch

    from oracle import attention as oracle
    from trident_amd import workloads

    q, k, v, d_o, mask = workloads.make_inputs(w)
    if mask is not None:
        mask = mask.to(w.dtype)
    times = []
    for rep in range(max(reps, 1) + (1 if reps > 0 else 0)):
        tq, tk, tv = [x.clone().requires_grad_(w.backward) for x in (q, k, v)]
        t0 = time.perf_counter()
        out = oracle.sdpa_cpu(tq, tk, tv, mask, w.dropout_p, w.is_causal)
        if w.backward:
            out.backward(d_o)
        dt = time.perf_counter() - t0
        if rep > 0 or reps == 0:
            times.append(dt)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": round(w.flops(w.backward) / med / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"torch CPU scaled_dot_product_attention, full {w.name} workload "
                  f"({'fwd+bwd' if w.backward else 'fwd'}), {'1 warm-up + ' + str(reps) + ' timed reps' if reps else 'one cold rep'}, median {med:.3f} s; "
                  f"os.cpu_count()={os.cpu_count()}",
    }


def config_figures(dev, with_cpu):
    """Forward and forward+backward figures of all five configurations (each with its own CPU baseline) and of the two
    extra workloads (C3's shape in fp32, a 16-bit problem with head size 32; no CPU baseline)."""
    from trident_amd import workloads

    out = {}
    for name, wl in {**workloads.WORKLOADS, **workloads.EXTRA_WORKLOADS}.items():
        pth = Path(wl, dev)
        # The CPU baseline before it left the GPU idle and its clock low: warm up with this configuration's own steps for
        # about 0.15 s (the clock needs tens of milliseconds of load), at least 8 steps, then time.
        rough, _ = run_steps(pth, 2, 1)
        warm = 2 if name == "C5" else max(8, min(4000, int(150.0 / max(rough, 1e-3))))
        ms, pk = run_steps(pth, 5 if name == "C5" else 30, warm)
        peak = PEAK_TFLOPS[_dtype_name(wl.dtype)]
        f = wl.flops() / (pk["fwd"] + pk.get("mask_classes", 0.0)) / 1e9  # (the classification belongs to the forward)
        row = {"workload": describe(wl), "fwd_tflops": round(f, 2), "fwd_frac_of_peak": round(f / peak, 4),
               "peak_tflops": peak, "kernel_ms": {k: round(v, 5) for k, v in pk.items()}}
        if wl.backward:
            t = wl.flops(True) / ms / 1e9
            row.update(fwdbwd_tflops=round(t, 2), fwdbwd_frac_of_peak=round(t / peak, 4), ms_per_step=round(ms, 5))
        if "bwd_delta" in pk:  # HBM-bound pre-pass: bytes it must move / its duration
            gbs = pth.algorithmic_bytes("bwd_delta") / pk["bwd_delta"] / 1e6
            row["delta_prepass"] = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                    "frac": round(gbs / HBM_PEAK_GBS, 4)}
        if wl.masked:  # mask streaming: every head reads its batch's S x S fp32 mask once per kernel
            B, H, S, _ = pth.q.shape
            logical, unique = 4.0 * B * H * S * S, 4.0 * B * S * S
            row["mask_stream"] = {k: {"logical_GBps": round(logical / pk[k] / 1e6, 1),
                                      "unique_GBps": round(unique / pk[k] / 1e6, 1)} for k in pk if k != "bwd_delta"}
            if not wl.dense_mask:
                lengths = (pth.mask[:, 0, 0] == 0).sum(-1)
                row["masked_key_fraction"] = round(1.0 - float(lengths.float().mean()) / S, 4)
            row["mask_stream"]["note"] = ("fp32 mask bytes every workgroup asks for (logical: B*H*S*S*4; unique: "
                                          "B*S*S*4, the heads of a batch share it) / kernel duration; HBM peak 8000 GB/s")
        if with_cpu and name in workloads.WORKLOADS:
            cb = cpu_baseline(wl, reps={"C3": 1, "C4": 1, "C5": 0}.get(name, 3))
            row.update(cpu_tflops=cb["value"], cpu_cores=cb["cores"])
        out[name] = row
        del pth
    return out


def sibling_ops(dev):
    """HBM-bound sibling operations through the operator API on one large input (bf16, 16384 x 8192 = 256 MiB):
    achieved bytes/s against the 8 TB/s HBM peak, algorithmic bytes = every tensor read or written once."""
    import torch

    import trident_amd
    from trident_amd import rowops

    y, x = 16384, 8192
    inp = torch.randn(y, x, device=dev).to(torch.bfloat16).requires_grad_(True)
    grad = torch.randn(y, x, device=dev).to(torch.bfloat16)
    mask = (torch.rand(y, x, device=dev) < 0.25).to(torch.uint8)
    nbytes = y * x * 2
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]

    def timed(fn, reps=10):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        ev[0].record()
        for _ in range(reps):
            fn()
        ev[1].record()
        torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[1]) / reps

    res = {"input": f"bf16 {y} x {x} (256 MiB), softmax along the rows; uint8 mask, 25 % set"}
    out = trident_amd.function.softmax(inp.detach(), 1)
    cases = [
        ("softmax_fwd", lambda: trident_amd.function.softmax(inp.detach(), 1), 2 * nbytes),
        ("softmax_bwd", lambda: rowops._softmax_backward(grad, out, 1, "kernel.Softmax.backward"), 3 * nbytes),
        ("masked_softmax_fwd", lambda: trident_amd.function.masked_softmax(inp.detach(), mask, 1), 2 * nbytes + y * x),
        ("dropout_fwd", lambda: trident_amd.function.dropout(inp.detach(), 0.1), 2 * nbytes),
    ]
    for name, fn, moved in cases:
        ms = timed(fn)
        gbs = moved / ms / 1e6
        res[name] = {"ms": round(ms, 4), "bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4)}
    return res


def reference_scenario(dev, mode, dtype_name):
    """The reference's own attention benchmark (benchmarks/benchmark_attention.py:20-57): forward at B=64, H=8, D=64 and
    backward at B=32, H=8, D=64, sequence lengths 32 ... 512, non-causal, no mask; milliseconds per call for this
    library, for torch's own GPU attention (the reference's 'torch' backend) and for torch on the host cores."""
    import torch

    import trident_amd

    dtype = {"float32": torch.float32, "float16": torch.float16, "bfloat16": torch.bfloat16}[dtype_name]
    B = 64 if mode == "forward" else 32
    H, D = 8, 64
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]

    def timed(fn, reps=100):
        for _ in range(20):  # (the first calls of a process also load the kernels' code objects)
            fn()
        torch.cuda.synchronize()
        ev[0].record()
        for _ in range(reps):
            fn()
        ev[1].record()
        torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[1]) / reps

    rows = []
    for S in [2**i for i in range(5, 10)]:
        g = torch.Generator().manual_seed(S)
        q, k, v, d_o = [torch.randn(B, H, S, D, generator=g).to(dtype) for _ in range(4)]
        flops = 4.0 * B * H * S * S * D * (1.0 if mode == "forward" else 2.5)
        row = {"y_size": S}
        for backend in ("trident_amd", "torch_gpu", "torch_cpu"):
            f = trident_amd.function.scaled_dot_product_attention if backend == "trident_amd" else \
                torch.nn.functional.scaled_dot_product_attention
            loc = "cpu" if backend == "torch_cpu" else dev
            tq, tk, tv = [x.to(loc).requires_grad_(mode != "forward") for x in (q, k, v)]
            tg = d_o.to(loc)
            if mode == "forward":
                call = lambda: f(tq, tk, tv)
            else:
                out = f(tq, tk, tv)
                call = lambda: out.backward(tg, retain_graph=True)
            if backend == "torch_cpu":
                call()
                t0 = time.perf_counter()
                for _ in range(3):
                    call()
                ms = (time.perf_counter() - t0) * 1e3 / 3
            else:
                ms = timed(call)
            row[backend + "_ms"] = round(ms, 4)
            row[backend + "_tflops"] = round(flops / ms / 1e9, 2)
        rows.append(row)
    return {"scenario": "attention " + mode, "num_batches": B, "num_heads": H, "x_size": D, "dtype": dtype_name,
            "cpu_threads": torch.get_num_threads(), "rows": rows,
            "note": "backward times output.backward(grad, retain_graph=True) as the reference's benchmark does (gradients "
                    "accumulate into .grad); flops: forward 4 B H S^2 D, backward 10 B H S^2 D"}


def ceiling(dev):
    """What the matrix pipe sustains on this box, in this process: MFMA-only loops on random operands (registers;
    A operands from LDS; every LDS read feeding two MFMAs), a large bf16 GEMM, and the three C3 attention kernels."""
    import torch

    from trident_amd import _lib, workloads

    probe = _lib.probe_lib()
    peak = PEAK_TFLOPS["bf16"]
    res = {"peak_tflops": peak, "operands": "bf16 N(0,1) random (torch.randn, seed 1)"}
    torch.manual_seed(1)
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    operands = torch.randn(16 * 512 * 8, device=dev).to(torch.bfloat16)
    out = torch.empty(cus * 512, device=dev, dtype=torch.float32)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]

    def timed(fn, reps):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        ev[0].record()
        for _ in range(reps):
            fn()
        ev[1].record()
        torch.cuda.synchronize()
        return ev[0].elapsed_time(ev[1]) / reps

    iters = 4000
    for mode, name in ((0, "mfma_registers"), (1, "mfma_lds_1_read_per_mfma"), (2, "mfma_lds_1_read_per_2_mfma")):
        ms = timed(lambda: _lib.check(probe.tri_probe_mfma(mode, cus, iters, operands.data_ptr(), out.data_ptr(),
                                                               torch.cuda.current_stream().cuda_stream)), 5)
        tf = cus * 8 * iters * 64 * 32768.0 / ms / 1e9
        res[name] = {"ms": round(ms, 3), "tflops": round(tf, 1), "frac_of_peak": round(tf / peak, 4),
                     "busy_x_clock_GHz": round(2.4 * tf / peak, 3)}
    ms = timed(lambda: _lib.check(probe.tri_probe_mfma(3, cus, iters // 4, operands.data_ptr(), out.data_ptr(),
                                                           torch.cuda.current_stream().cuda_stream)), 5)
    tf = cus * 8 * (iters // 4) * 64 * 4096.0 / ms / 1e9
    res["mfma_fp32_registers"] = {"ms": round(ms, 3), "tflops": round(tf, 1), "peak_tflops": PEAK_TFLOPS["fp32"],
                                  "frac_of_peak": round(tf / PEAK_TFLOPS["fp32"], 4),
                                  "busy_x_clock_GHz": round(2.4 * tf / PEAK_TFLOPS["fp32"], 3)}
    # vector work of one wave beside another wave's MFMAs on the same SIMD: alone, alone, together (ms)
    co = {}
    for matrix, mname in ((0, "bf16_32x32x16"), (1, "fp32_32x32x2")):
        for valu, vname in ((0, "fma"), (1, "exp2"), (2, "fma_max_exp2")):
            row = {}
            for who, wname in ((1, "matrix_ms"), (2, "vector_ms"), (3, "both_ms"), (4, "same_wave_ms")):
                row[wname] = round(timed(lambda: _lib.check(probe.tri_probe_coexec(
                    matrix, valu, who, cus, 2000, operands.data_ptr(), out.data_ptr(),
                    torch.cuda.current_stream().cuda_stream)), 3), 3)
            row["hidden_fraction_of_vector_work"] = round((row["matrix_ms"] + row["vector_ms"] - row["both_ms"]) / row["vector_ms"], 3)
            row["hidden_fraction_same_wave"] = round((row["matrix_ms"] + row["vector_ms"] - row["same_wave_ms"]) / row["vector_ms"], 3)
            co[mname + "+" + vname] = row
    res["coexecution"] = co
    n = 8192
    a = torch.randn(n, n, device=dev).to(torch.bfloat16)
    b = torch.randn(n, n, device=dev).to(torch.bfloat16)
    ms = timed(lambda: torch.matmul(a, b), 20)
    tf = 2.0 * n**3 / ms / 1e9
    res["torch_matmul_8192_bf16"] = {"ms": round(ms, 3), "tflops": round(tf, 1), "frac_of_peak": round(tf / peak, 4)}
    del a, b
    pth = Path(workloads.WORKLOADS["C3"], dev)
    _, pk = run_steps(pth, 30, 5)
    executed = {"fwd": 4.0 * 36 / 32, "bwd_dq": 6.0, "bwd_dkdv": 8.0 * 34 / 32}  # units of B H S^2 D / 2 the kernels run
    unit = pth.w.flops() / 4.0
    res["c3_kernels"] = {k: {"ms": round(v, 4), "credited_tflops": round(pth.algorithmic_flops(k) / v / 1e9, 1),
                             "executed_tflops": round(executed[k] * unit / v / 1e9, 1),
                             "executed_frac_of_peak": round(executed[k] * unit / v / 1e9 / peak, 4)}
                        for k, v in pk.items() if k in executed}
    # If vector work beside MFMAs costs its full time (coexecution above: hidden fraction about 0 under sustained load), a
    # kernel cannot be faster than its MFMAs at the LDS-fed rate plus its per-score vector work (one fma, max, exp2 mix per
    # score, the probe's rate: 256 lanes x 32 values x 2000 trips per CU in vector_ms).
    w = pth.w
    scores = w.B * w.H * w.S * w.S * (0.5 if w.is_causal else 1.0)
    mix = co["bf16_32x32x16+fma_max_exp2"]
    vec_ms = scores * mix["vector_ms"] / (cus * 256 * 32 * 2000.0)
    for k in res["c3_kernels"]:
        mfma_ms = executed[k] * unit / (res["mfma_lds_1_read_per_mfma"]["tflops"] * 1e9)
        row = res["c3_kernels"][k]
        row["additive_floor_ms"] = round(mfma_ms + vec_ms, 4)
        row["floor_over_measured"] = round((mfma_ms + vec_ms) / row["ms"], 3)
    return res


def sustained_clock(dev, seconds=1.5):
    """The C3 step under sustained load with its seeded random operands and with all-zero operands (same launches, same
    cycle counts): milliseconds per step and the shader clock and board power sampled meanwhile (torch.cuda.clock_rate /
    power_draw, every 50 ms, second half of the run). The clock this load sustains depends on the operand bits, i.e. on
    the power the matrix pipe draws: that, not the 2.4 GHz the published peak assumes, is what the kernels run at."""
    import threading

    import torch

    from trident_amd import workloads

    w = workloads.WORKLOADS["C3"]
    res = {"workload": describe(w), "seconds_per_case": seconds}
    for label in ("random_operands", "zero_operands", "random_operands_again"):
        path = Path(w, dev)
        if label == "zero_operands":
            for t in (path.q, path.k, path.v, path.d_o):
                t.zero_()
        samples, stop = [], [False]

        def sampler():
            while not stop[0]:
                try:
                    samples.append((float(torch.cuda.clock_rate(dev)), float(torch.cuda.power_draw(dev))))
                except Exception:  # (no management library on this box: the timing still stands)
                    return
                time.sleep(0.05)

        th = threading.Thread(target=sampler)
        th.start()
        n, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for _ in range(50):
                for _, fn in path.kernels:
                    fn()
            torch.cuda.synchronize()
            n += 50
        dt = time.perf_counter() - t0
        stop[0] = True
        th.join()
        tail = samples[len(samples) // 2:]
        row = {"ms_per_step": round(dt / n * 1e3, 5), "tflops": round(w.flops(True) / (dt / n) / 1e12, 1), "samples": len(tail)}
        if tail:
            row["clock_mhz"] = round(sum(x[0] for x in tail) / len(tail))
            row["power_draw_raw"] = round(sum(x[1] for x in tail) / len(tail))
        res[label] = row
        del path
    return res


def describe(w):
    extra = "causal" if w.is_causal else (("dense " if w.dense_mask else "") + "additive fp32 mask [B,1,S,S]" if w.masked else "plain")
    if w.dropout_p:
        extra += f" dropout {w.dropout_p}"
    return f"{w.name}: {_dtype_name(w.dtype)} {extra} B={w.B} H={w.H} S={w.S} D={w.D} {'fwd+bwd' if w.backward else 'fwd'}"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="C3")
    ap.add_argument("--report", action="store_true", help="also print all five configurations on stderr")
    ap.add_argument("--no-configs", action="store_true", help="leave the five-configuration table out of the JSON line")
    ap.add_argument("--scenario", choices=["attention"], help="instead of the benchmark: the reference's benchmark scenario "
                    "(benchmarks/benchmarker.py --scenario attention), one JSON line")
    ap.add_argument("--mode", choices=["forward", "backward"], default="forward")
    ap.add_argument("--dtype", choices=["float32", "float16", "bfloat16"], default="float32")
    ap.add_argument("--sibling-ops", action="store_true", help="instead of the benchmark: one JSON line with the HBM-bound "
                    "sibling operations (softmax forward/backward, masked softmax, dropout)")
    ap.add_argument("--ceiling", action="store_true",
                    help="instead of the benchmark: print one JSON line with the MFMA ceiling of this box (random-operand "
                         "MFMA loops, a bf16 GEMM, the C3 kernels)")
    ap.add_argument("--sustained-clock", action="store_true",
                    help="instead of the benchmark: one JSON line with the C3 step under sustained load, its seeded random "
                         "operands against all-zero operands, and the shader clock sampled meanwhile")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (known HBM traffic) so that rocprofv3 FETCH_SIZE / "
                         "WRITE_SIZE readings of the attention kernels can be scaled against it")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs on one GPU; the attention path has no exchange step to "
                 "measure across GPUs (heads shard independently). Run with --gpus 1.")

    import torch

    from trident_amd import workloads

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    w = {**workloads.WORKLOADS, **workloads.EXTRA_WORKLOADS}[a.workload]
    if a.ceiling:
        print(json.dumps({"ceiling": ceiling(dev)}), flush=True)
        return
    if a.sustained_clock:
        print(json.dumps({"sustained_clock": sustained_clock(dev)}), flush=True)
        return
    if a.sibling_ops:
        print(json.dumps({"sibling_ops": sibling_ops(dev)}), flush=True)
        return
    if a.scenario:
        print(json.dumps({"reference_scenario": reference_scenario(dev, a.mode, a.dtype)}), flush=True)
        return
    if a.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    path = Path(w, dev)
    flops_step = w.flops(w.backward)
    # right after start-up, on a clock that is still rising from idle: reported, not the headline
    cold_ms, _ = run_steps(path, a.steps, a.warmup)
    extras = {"cold_start": {"ms_per_step": round(cold_ms, 5), "tflops": round(flops_step / cold_ms / 1e9, 1),
                             "note": "the same W + K steps as the first GPU work of the process, before the clock has settled"}}
    if not a.no_cpu:
        extras["cpu_baseline"] = cpu_baseline(w)
    if not a.no_configs:
        for key, leg in (("configs", lambda: config_figures(dev, not a.no_cpu)), ("sibling_ops", lambda: sibling_ops(dev))):
            try:
                extras[key] = leg()
            except Exception as e:  # (the headline below must not depend on the other legs)
                extras[key] = {"error": f"{type(e).__name__}: {e}"}
    op_steps, op_warmup = max(a.steps, 100), max(a.warmup, 20)
    op_ms = operator_ms(w, dev, op_steps, op_warmup)
    extras["operator_api"] = {"ms_per_step": round(op_ms, 5), "tflops": round(flops_step / op_ms / 1e9, 1), "steps": op_steps,
                              "warmup": op_warmup, "note": "same step through function.scaled_dot_product_attention + autograd"}
    # the headline region, directly after sustained load on the same workload
    wall_ms, per_kernel = run_steps(path, a.steps, a.warmup)
    dname = _dtype_name(w.dtype)
    peak = PEAK_TFLOPS[dname]
    value = flops_step / wall_ms / 1e9
    fwd_tf = w.flops() / (per_kernel["fwd"] + per_kernel.get("mask_classes", 0.0)) / 1e9

    dominant = max(per_kernel, key=per_kernel.get)
    dom_flops = path.algorithmic_flops(dominant)
    achieved = dom_flops / per_kernel[dominant] / 1e9
    roofline = {
        "kernel": dominant,
        "bound": "mfma",
        "achieved": round(achieved, 1),
        "peak": peak,
        "unit": "TFLOP/s",
        "frac": round(achieved / peak, 4),
        "traffic": measured_traffic(w.name, dominant),
        "avg_launch_ms": round(per_kernel[dominant], 5),
    }
    result = {
        "metric": ("attention fwd & fwd+bwd TFLOP/s + % MFMA peak, bf16 causal S=4096 D=128" if w.name == "C3" else
                   "attention " + ("fwd+bwd" if w.backward else "fwd") + " TFLOP/s + % MFMA peak, " + describe(w)),
        "value": round(value, 1),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dname,
        "data": "synthetic",
        "config": {"workload": describe(w)},
        "fwd_tflops": round(fwd_tf, 1),
        "fwd_frac_of_peak": round(fwd_tf / peak, 4),
        "fwdbwd_tflops": round(value, 1),
        "fwdbwd_frac_of_peak": round(value / peak, 4),
        "kernel_ms": {k: round(v, 5) for k, v in per_kernel.items()},
        "roofline": roofline,
    }
    if "bwd_delta" in per_kernel:
        nbytes = path.algorithmic_bytes("bwd_delta")
        gbs = nbytes / per_kernel["bwd_delta"] / 1e6
        result["delta_prepass"] = {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                   "frac": round(gbs / HBM_PEAK_GBS, 4)}
    result.update(extras)
    print(json.dumps(result), flush=True)

    if a.report:
        for name, wl in workloads.WORKLOADS.items():
            pth = Path(wl, dev)
            steps = 3 if name == "C5" else 10
            ms, pk = run_steps(pth, steps, 2)
            pkk = PEAK_TFLOPS[_dtype_name(wl.dtype)]
            f = wl.flops() / pk["fwd"] / 1e9
            line = f"{describe(wl)} | fwd {pk['fwd']:.4f} ms {f:.1f} TFLOP/s ({100 * f / pkk:.1f}% of {pkk})"
            if wl.backward:
                t = wl.flops(True) / ms / 1e9
                line += f" | fwd+bwd {ms:.4f} ms {t:.1f} TFLOP/s ({100 * t / pkk:.1f}%)"
                line += " | " + " ".join(f"{k}={v:.4f}ms" for k, v in pk.items())
            if not a.no_cpu and name != "C5":
                cb = cpu_baseline(wl, reps=1 if name in ("C3", "C4") else 3)
                line += f" | CPU {cb['value']} TFLOP/s on {cb['cores']} threads"
            print(line, file=sys.stderr, flush=True)
            del pth


if __name__ == "__main__":
    main()
