#!/usr/bin/env python3
"""Benchmark of the BTP hot path: forward + backward at B=1024, L=128, dim=512 (H=32) bf16.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c3|c4|c5|r2032|r64|r192] [--no-cpu-baseline] [--no-other-configs]

A step is one forward plus one backward launch through the C ABI on one batch of synthetic
input that is already resident in HBM. Buffers rotate over several independent sets so that a
step never finds its inputs in the 256 MiB last-level cache left there by the previous step.
Prints ONE JSON line (see the keys below).

Algorithmic bytes per (token, head): forward 66 (coeff 2 + x 32 read, y 32 written), backward 102
(coeff 2 + x 32 + dy 32 read, dx 32 + dA 4 written), together 168; per token multiply by H.
"""

from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X HBM3E, published peak
FWD_BYTES, BWD_BYTES = 66, 102  # per (token, head), bf16 y / dy

PROFILES = os.path.join(ROOT, "profiles")


def profiled_traffic(config, kernel):
    """HBM bytes per launch of `kernel` at workload `config`, as rocprofv3 counted them: the 'total MB' column of the
    kernel's row in the 'HBM traffic per dispatch' table of profiles/btp_kernels_<config>_*.txt (FETCH_SIZE and
    WRITE_SIZE, each scaled by what the same counter reads for the copy kernel; the commands are in that file).
    Counters cannot be read from inside this script, so the committed summary is the source; returns
    (bytes, source) or (None, None) when there is no such file or row."""
    import glob
    import re

    for path in sorted(glob.glob(os.path.join(PROFILES, f"btp_kernels_{config}_*.txt"))):
        in_table, column = False, None
        with open(path, encoding="utf-8") as fh:
            for line in fh:
                if line.startswith("== "):
                    in_table = line.startswith("== HBM traffic per dispatch")
                    column = None
                    continue
                if not in_table:
                    continue
                if line.startswith("kernel ") and "total MB" in line:
                    # columns after the name: read KiB, alg read, written KiB, alg written, total MB, ratio
                    column = -2
                    continue
                m = re.match(r"^(\S.*?)\s{2,}([-+0-9.eE\s]+)$", line.rstrip())
                if column is not None and m and m.group(1) == kernel:
                    fields = m.group(2).split()
                    if len(fields) == 6:
                        rel = os.path.relpath(path, ROOT)
                        return float(fields[column]) * 1e6, {"file": rel, "table": "HBM traffic per dispatch",
                                                              "row": kernel, "column": "total MB"}
    return None, None


CONFIGS = {
    # name: (B, H, L, seed, x_std, gate)
    "c3": (1024, 32, 128, 1234, 0.25, "sigmoid"),
    "c4": (16, 64, 8192, 1235, 0.25, "sigmoid"),
    "c5": (64, 128, 2048, 1236, 1.0, "mixed"),
    # not one of the reference's benchmark shapes: c5's size with rows of 4064 bytes, which do not end on a 128-byte
    # cache line (the stand-alone kernels move such rows as whole lines and pass row ends between wavefronts)
    "r2032": (64, 128, 2032, 1237, 0.25, "sigmoid"),
    # rows that would leave a span of 128 steps partly empty: the kernels cut spans from the blocks of all rows in order
    # (rows of 64 steps share a wavefront two by two; rows of 192 steps start anywhere in one)
    "r64": (2048, 32, 64, 1238, 0.25, "sigmoid"),
    "r192": (1024, 32, 192, 1239, 0.25, "sigmoid"),
}
LAYER_LAYOUT_CONFIGS = ("c3", "c4", "c5")  # the fused kernels' rows are feature vectors: L does not change their alignment


def synth(B, H, L, seed, x_std, gate):
    import torch

    g = torch.Generator(device="cpu").manual_seed(seed)
    x = (torch.randn(B, H, 16, L, generator=g) * x_std).to(torch.bfloat16)
    if gate == "sigmoid":
        coeff = torch.exp(-torch.nn.functional.softplus(torch.randn(B, H, L, generator=g)))
    else:
        forget = torch.rand(B, H, 1, generator=g) < 0.5
        lo = -20.0 + 15.0 * torch.rand(B, H, L, generator=g)
        hi = -1e-4 * torch.rand(B, H, L, generator=g)
        coeff = torch.exp(torch.where(forget, lo, hi))
    dy = torch.randn(B, H, 16, L, generator=g).to(torch.bfloat16)
    return coeff.to(torch.bfloat16), x, dy


def cpu_baseline(B, H, L, seed, x_std, gate, budget_s=20.0):
    """Times the PyTorch restatement of the reference's CPU path (block_two_pass_log, forward +
    backward through autograd, bf16 tensors) on a bounded sample of the workload's batch."""
    import torch

    from spear_amd.ops.btp.reference import block_two_pass_log

    threads = torch.get_num_threads()

    def once(bs):
        coeff, x, dy = synth(bs, H, L, seed, x_std, gate)
        coeff.requires_grad_(True)
        x.requires_grad_(True)
        t0 = time.perf_counter()
        y = block_two_pass_log(coeff, x, 16)
        y.backward(dy)
        return time.perf_counter() - t0

    once(max(1, min(B, 4)))  # warm-up (thread pool, allocator)
    bs, t = max(1, min(B, 8)), 0.0
    while True:  # grow the sample until one run is long enough to extrapolate from
        t = once(bs)
        if t >= 0.5 or bs >= B:
            break
        bs = min(B, bs * 4)
    bs = int(max(1, min(B, bs * (budget_s / 4.0) / max(t, 1e-6))))
    reps = 3
    times = [once(bs) for _ in range(reps)]
    while sum(times) < budget_s / 2.0 and len(times) < 41:  # whole batch already fits: repeat instead
        times.append(once(bs))
    reps = len(times)
    med = statistics.median(times)
    return {
        "value": bs * L / med,
        "unit": "tokens/s",
        "cores": threads,
        "kind": "port",
        "sample": f"block_two_pass_log fwd+bwd (autograd), bf16, first {bs} of {B} batch rows, H={H}, L={L}; median of {reps} runs after 1 warm-up; {med:.3f} s per run, {sum(times):.1f} s timed",
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", choices=sorted(CONFIGS), default="c3")
    ap.add_argument("--sets", type=int, default=8, help="independent buffer sets to rotate over")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-fused", action="store_true", help="skip the fused layer-layout forward leg")
    ap.add_argument("--no-streaming", action="store_true", help="skip the prefill / decode-step leg")
    ap.add_argument("--no-layer", action="store_true", help="skip the whole-layer (projections + mixing) leg")
    ap.add_argument("--no-other-configs", action="store_true", help="skip the legs at the other full-size configurations")
    ap.add_argument("--settle-seconds", type=float, default=0.3, help="untimed run-in before the warm-up steps")
    args = ap.parse_args()

    if args.gpus != 1:
        print(
            "bench.py: this build measures one GPU only (the op shards over batch and heads with no "
            "communication, so N GPUs run N independent copies of the same kernel). Run with --gpus 1.",
            file=sys.stderr,
        )
        return 2

    import torch

    from spear_amd import _btp

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    lib = _btp.load_library()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    B, H, L, seed, x_std, gate = CONFIGS[args.config]
    coeff, x, dy = synth(B, H, L, seed, x_std, gate)
    sets = []
    for _ in range(args.sets):
        s = {
            "coeff": coeff.to(dev),
            "x": x.to(dev),
            "dy": dy.to(dev),
            "y": torch.empty(B, H, 16, L, device=dev, dtype=torch.bfloat16),
            "dx": torch.empty(B, H, 16, L, device=dev, dtype=torch.bfloat16),
            "dA": torch.empty(B, H, L, device=dev, dtype=torch.float32),
        }
        sets.append(s)
    del coeff, x, dy
    stream = torch.cuda.current_stream(dev)
    sp = ctypes.c_void_p(stream.cuda_stream)

    def fwd(s):
        rc = lib.spear_btp_forward(s["coeff"].data_ptr(), s["x"].data_ptr(), s["y"].data_ptr(), None,
                                   B, H, L, 2, 0, 0, 0, sp)
        assert rc == 0, lib.spear_btp_last_error()

    def bwd(s):
        rc = lib.spear_btp_backward(s["coeff"].data_ptr(), s["x"].data_ptr(), s["dy"].data_ptr(), None,
                                    s["dx"].data_ptr(), s["dA"].data_ptr(), B, H, L, 2, 0, 0, 0, sp)
        assert rc == 0, lib.spear_btp_last_error()

    def step(i):
        s = sets[i % len(sets)]
        fwd(s)
        bwd(s)

    # Untimed: let clocks and power state settle (about 0.3 s of steps), then the W warm-up steps.
    t_settle = time.perf_counter()
    i = 0
    while time.perf_counter() - t_settle < args.settle_seconds:
        step(i)
        i += 1
        if i % 64 == 0:
            torch.cuda.synchronize()
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()

    # Timed region: exactly K steps, synchronised on both sides; HIP events on the launch stream
    # bracket the same region to give the device-side duration.
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)
    for i in range(args.steps):
        step(i)
    ev1.record(stream)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed * 1e3 / args.steps
    ms_per_step_device = ev0.elapsed_time(ev1) / args.steps

    # per-kernel average launch duration, HIP events on the launch stream, same rotation
    def kernel_ms(fn):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(min(args.warmup, 10)):
            fn(sets[i % len(sets)])
        torch.cuda.synchronize()
        e0.record(stream)
        for i in range(args.steps):
            fn(sets[i % len(sets)])
        e1.record(stream)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / args.steps

    fwd_ms, bwd_ms = kernel_ms(fwd), kernel_ms(bwd)

    # spread of single steps: one event pair per step (adds the event cost to each sample, so these
    # sit slightly above ms_per_step_device; they show the run-to-run spread, not the headline)
    def step_spread():
        n = min(args.steps, 200)
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
        evs[0].record(stream)
        for i in range(n):
            step(i)
            evs[i + 1].record(stream)
        torch.cuda.synchronize()
        d = sorted(evs[i].elapsed_time(evs[i + 1]) for i in range(n))
        pick = lambda q: d[min(n - 1, int(q * n))]
        return {"samples": n, "p10_ms": pick(0.10), "median_ms": pick(0.50), "p90_ms": pick(0.90)}

    spread = step_spread()

    def fwd_mfma(s):  # same op through the bf16-MFMA tile kernel, for comparison
        rc = lib.spear_btp_forward(s["coeff"].data_ptr(), s["x"].data_ptr(), s["y"].data_ptr(), None,
                                   B, H, L, 2, 0, 0, 2, sp)
        assert rc == 0, lib.spear_btp_last_error()

    def bwd_mfma(s):  # the backward on the matrix cores (three 16x16x32 products per block)
        rc = lib.spear_btp_backward(s["coeff"].data_ptr(), s["x"].data_ptr(), s["dy"].data_ptr(), None,
                                    s["dx"].data_ptr(), s["dA"].data_ptr(), B, H, L, 2, 0, 0, 2, sp)
        assert rc == 0, lib.spear_btp_last_error()

    fwd_mfma_ms, bwd_mfma_ms = kernel_ms(fwd_mfma), kernel_ms(bwd_mfma)

    # copy kernel of the same footprint as a practical ceiling (reads n, writes n)
    nbytes = sets[0]["x"].numel() * 2
    def copy(s):
        lib.spear_btp_copy(s["x"].data_ptr(), s["dx"].data_ptr(), ctypes.c_ulonglong(nbytes), sp)
    copy_ms = kernel_ms(copy)

    # the operator's own access shape and cache policy without its arithmetic: 4 KiB per wavefront,
    # non-temporal loads and stores; one input (copy) and two inputs (the backward kernel's mix)
    def probe_copy(s):
        rc = lib.spear_btp_stream_probe(s["x"].data_ptr(), None, s["dx"].data_ptr(), ctypes.c_ulonglong(nbytes), sp)
        assert rc == 0, lib.spear_btp_last_error()

    def probe_2r1w(s):
        rc = lib.spear_btp_stream_probe(s["x"].data_ptr(), s["dy"].data_ptr(), s["dx"].data_ptr(),
                                        ctypes.c_ulonglong(nbytes), sp)
        assert rc == 0, lib.spear_btp_last_error()

    probe_copy_ms, probe_2r1w_ms = kernel_ms(probe_copy), kernel_ms(probe_2r1w)
    ceil_copy = 2 * nbytes / (probe_copy_ms * 1e-3) / 1e9
    ceil_2r1w = 3 * nbytes / (probe_2r1w_ms * 1e-3) / 1e9

    # the same traffic in other launch shapes: is there a shape the kernels could borrow that moves more?
    shape_names = ["one_slab_per_wave", "two_slabs_per_wave", "loop_4_slabs_prefetch", "persistent_grid_prefetch",
                   "one_16B_element_per_thread"]
    probe_shapes = {}
    for shape, name in enumerate(shape_names):
        def shaped(s, second, shape=shape):
            rc = lib.spear_btp_stream_probe_shape(s["x"].data_ptr(), s["dy"].data_ptr() if second else None,
                                                  s["dx"].data_ptr(), ctypes.c_ulonglong(nbytes), shape, sp)
            assert rc == 0, lib.spear_btp_last_error()
        t1, t2 = kernel_ms(lambda s: shaped(s, False)), kernel_ms(lambda s: shaped(s, True))
        probe_shapes[name] = {"copy_1r1w": 2 * nbytes / (t1 * 1e-3) / 1e9, "nt_2r1w": 3 * nbytes / (t2 * 1e-3) / 1e9}
    best_copy = max(v["copy_1r1w"] for v in probe_shapes.values())
    best_2r1w = max(v["nt_2r1w"] for v in probe_shapes.values())

    # one direction at a time: HBM serves reads and writes one after the other, so a kernel that reads R bytes
    # and writes W bytes takes at least R / read_rate + W / write_rate; this is the floor the kernels are up against
    def one_way(shape, second):
        def fn(s):
            rc = lib.spear_btp_stream_probe_shape(s["x"].data_ptr(), s["dy"].data_ptr() if second else None,
                                                  s["dx"].data_ptr(), ctypes.c_ulonglong(nbytes), shape, sp)
            assert rc == 0, lib.spear_btp_last_error()
        return kernel_ms(fn)
    read_rate = 2 * nbytes / (one_way(5, True) * 1e-3) / 1e9
    write_rate = nbytes / (one_way(6, False) * 1e-3) / 1e9
    def serial_floor(read_bytes, write_bytes):  # GB/s of algorithmic bytes if reads and writes just add up
        return (read_bytes + write_bytes) / (read_bytes / read_rate + write_bytes / write_rate)
    floor_fwd, floor_bwd = serial_floor(34, 32), serial_floor(66, 36)
    # the 2R:1W probe with a compute phase of the backward kernel's length (640 dependent FMAs) between loads and stores
    with_compute_2r1w = 3 * nbytes / (one_way(7, True) * 1e-3) / 1e9

    # log-space gate entry points on the same shape (fp32 gate in, fp32 dgate out: 68 + 108 B per unit)
    for s_ in sets:
        s_["gate"] = torch.log(s_["coeff"].float()).contiguous()

    def fwd_log(s):
        rc = lib.spear_btp_forward_loggate(s["gate"].data_ptr(), s["x"].data_ptr(), s["y"].data_ptr(), None,
                                           B, H, L, 2, 0, 0, 0, sp)
        assert rc == 0, lib.spear_btp_last_error()

    def bwd_log(s):
        rc = lib.spear_btp_backward_loggate(s["gate"].data_ptr(), s["x"].data_ptr(), s["dy"].data_ptr(),
                                            s["dx"].data_ptr(), s["dA"].data_ptr(), B, H, L, 2, 0, 0, 0, sp)
        assert rc == 0, lib.spear_btp_last_error()

    fwd_log_ms, bwd_log_ms = kernel_ms(fwd_log), kernel_ms(bwd_log)

    # the op's default types: btp(coeff, x) returns fp32 y and autograd hands back an fp32 dy (98 + 134 B per unit)
    for s_ in sets:
        s_["y32"] = torch.empty(B, H, 16, L, device=dev, dtype=torch.float32)

    def fwd_f32(s):
        rc = lib.spear_btp_forward(s["coeff"].data_ptr(), s["x"].data_ptr(), s["y32"].data_ptr(), None,
                                   B, H, L, 2, 0, 2, 0, sp)
        assert rc == 0, lib.spear_btp_last_error()

    def bwd_f32(s):  # y32 stands in for an fp32 dy: same bytes moved, values do not matter for the time
        rc = lib.spear_btp_backward(s["coeff"].data_ptr(), s["x"].data_ptr(), s["y32"].data_ptr(), None,
                                    s["dx"].data_ptr(), s["dA"].data_ptr(), B, H, L, 2, 0, 2, 0, sp)
        assert rc == 0, lib.spear_btp_last_error()

    fwd_f32_ms = kernel_ms(fwd_f32)
    bwd_f32_ms = kernel_ms(bwd_f32)

    # what the memory system gives the forward's 1 read : 2 writes (x in, an fp32 y out) in the kernels' launch shape,
    # without and with a compute phase (spear_btp_stream_probe_mix, x -> the two halves of y32)
    def probe_1r2w(compute):
        def fn(s):
            src = (ctypes.c_void_p * 1)(s["x"].data_ptr())
            dst = (ctypes.c_void_p * 2)(s["y32"].data_ptr(), s["y32"].data_ptr() + nbytes)
            rc = lib.spear_btp_stream_probe_mix(src, 1, dst, 2, ctypes.c_ulonglong(nbytes), compute, sp)
            assert rc == 0, lib.spear_btp_last_error()
        return 3 * nbytes / (kernel_ms(fn) * 1e-3) / 1e9
    ceil_1r2w = [probe_1r2w(0), probe_1r2w(1)]
    for s_ in sets:
        del s_["y32"]

    # fused layer-layout forward (gates + recurrence + y*C+V on [B, L, features] tensors) against the
    # same stage built from PyTorch ops around the stand-alone kernel
    def guarded(leg):
        """Run an auxiliary leg; if it raises, the headline measurement above still gets reported."""
        try:
            return leg()
        except Exception as exc:  # noqa: BLE001 - reported in the JSON line instead of propagating
            torch.cuda.synchronize()
            return {"error": f"{type(exc).__name__}: {exc}"}

    def fused_leg():
        from spear_amd.ops.btp import btp as btp_op

        F = H * 16
        g = torch.Generator(device="cpu").manual_seed(seed + 7)
        msets = []
        for _ in range(min(len(sets), 4)):
            msets.append({
                "a": torch.randn(B, L, H, generator=g).to(torch.bfloat16).to(dev),
                "b": torch.randn(B, L, F, generator=g).to(torch.bfloat16).to(dev),
                "c": torch.randn(B, L, F, generator=g).to(torch.bfloat16).to(dev),
                "v": torch.randn(B, L, F, generator=g).to(torch.bfloat16).to(dev),
                "out": torch.empty(B, L, F, device=dev, dtype=torch.bfloat16),
                "dout": torch.randn(B, L, F, generator=g).to(torch.bfloat16).to(dev),
                "da": torch.empty(B, L, H, device=dev, dtype=torch.bfloat16),
                "db": torch.empty(B, L, F, device=dev, dtype=torch.bfloat16),
                "dc": torch.empty(B, L, F, device=dev, dtype=torch.bfloat16),
                "dv": torch.empty(B, L, F, device=dev, dtype=torch.bfloat16),
            })

        def mix(s):
            rc = lib.spear_phalanx_mix_forward(s["a"].data_ptr(), s["b"].data_ptr(), s["c"].data_ptr(),
                                               s["v"].data_ptr(), s["out"].data_ptr(), B, L, H, H, 0, 0, sp)
            assert rc == 0, lib.spear_btp_last_error()

        def mix_bwd(s):
            rc = lib.spear_phalanx_mix_backward(s["a"].data_ptr(), s["b"].data_ptr(), s["c"].data_ptr(),
                                                s["v"].data_ptr(), s["dout"].data_ptr(), s["da"].data_ptr(),
                                                s["db"].data_ptr(), s["dc"].data_ptr(), s["dv"].data_ptr(),
                                                B, L, H, H, 0, 0, sp)
            assert rc == 0, lib.spear_btp_last_error()

        def unfused_stage(a, b, c, v):  # what the layer does around the stand-alone kernel (swr.py)
            A = torch.sigmoid(a).transpose(1, 2)
            V = v.transpose(1, 2).view(B, H, 16, L)
            X = torch.sigmoid(b).transpose(1, 2).view(B, H, 16, L) * V
            y = btp_op(A, X, 2, 32, torch.bfloat16) * c.transpose(1, 2).view(B, H, 16, L) + V
            return y.permute(0, 3, 1, 2).reshape(B, L, F)

        def mix_unfused(s):
            with torch.no_grad():
                s["out"].copy_(unfused_stage(s["a"], s["b"], s["c"], s["v"]))

        def mix_unfused_train(s):  # forward + backward through autograd
            leaves = [s[k].detach().requires_grad_(True) for k in ("a", "b", "c", "v")]
            unfused_stage(*leaves).backward(s["dout"])

        def kernel_ms_over(fn, pool):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            for i in range(5):
                fn(pool[i % len(pool)])
            torch.cuda.synchronize()
            n = max(20, args.steps // 4)
            e0.record(stream)
            for i in range(n):
                fn(pool[i % len(pool)])
            e1.record(stream)
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / n

        # the same kernels in q/k/v/gate terms: fp32 log-decay gate, out = q * btp(exp(gate), k * v) + v,
        # gradients dq, dk, dv and fp32 dgate; time-major [B, L, H, 16] tensors
        for s_ in msets:
            s_["gate"] = (-torch.nn.functional.softplus(s_["a"].float())).contiguous()
            s_["dgate"] = torch.empty(B, L, H, device=dev, dtype=torch.float32)
        QKV = 0x1

        def qkv(s):
            rc = lib.spear_phalanx_mix_forward(s["gate"].data_ptr(), s["b"].data_ptr(), s["c"].data_ptr(),
                                               s["v"].data_ptr(), s["out"].data_ptr(), B, L, H, H, 0, QKV, sp)
            assert rc == 0, lib.spear_btp_last_error()

        def qkv_bwd(s):
            rc = lib.spear_phalanx_mix_backward(s["gate"].data_ptr(), s["b"].data_ptr(), s["c"].data_ptr(),
                                                s["v"].data_ptr(), s["dout"].data_ptr(), s["dgate"].data_ptr(),
                                                s["db"].data_ptr(), s["dc"].data_ptr(), s["dv"].data_ptr(),
                                                B, L, H, H, 0, QKV, sp)
            assert rc == 0, lib.spear_btp_last_error()

        qkv_ms, qkv_bwd_ms = kernel_ms_over(qkv, msets), kernel_ms_over(qkv_bwd, msets)
        qkv_bytes = B * L * H * (4 + 3 * 32 + 32)             # gate, q, k, v read; out written
        qkv_bwd_bytes = B * L * H * (4 + 4 * 32 + 4 + 3 * 32)  # gate, q, k, v, dout read; dgate, dq, dk, dv written

        mix_ms, unfused_ms = kernel_ms_over(mix, msets), kernel_ms_over(mix_unfused, msets)
        mix_bwd_ms, unfused_train_ms = kernel_ms_over(mix_bwd, msets), kernel_ms_over(mix_unfused_train, msets)

        # what the memory system gives these stream counts in its best shape (contiguous 4 KiB pieces, short-lived
        # wavefronts, nothing shared): 3 inputs -> 1 output (forward) and 4 inputs -> 3 outputs (backward), without
        # and with a compute phase between the loads and the stores
        big = B * L * F * 2
        def mix_probe(n_src, n_dst, compute):
            def fn(s):
                src = (ctypes.c_void_p * n_src)(*[s[k].data_ptr() for k in ("b", "c", "v", "dout")[:n_src]])
                dst = (ctypes.c_void_p * n_dst)(*[s[k].data_ptr() for k in ("db", "dc", "dv")[:n_dst]])
                rc = lib.spear_btp_stream_probe_mix(src, n_src, dst, n_dst, ctypes.c_ulonglong(big), compute, sp)
                assert rc == 0, lib.spear_btp_last_error()
            return (n_src + n_dst) * big / (kernel_ms_over(fn, msets) * 1e-3) / 1e9
        ceil_fwd, ceil_fwd_c = mix_probe(3, 1, 0), mix_probe(3, 1, 1)
        ceil_bwd, ceil_bwd_c = mix_probe(4, 3, 0), mix_probe(4, 3, 1)
        mix_bytes = B * L * H * (2 + 3 * 32 + 32)          # a, b, c, v read; out written
        mix_bwd_bytes = B * L * H * (2 + 4 * 32 + 2 + 3 * 32)  # a, b, c, v, dout read; da, db, dc, dv written
        fused = {
            "avg_launch_ms": mix_ms, "algorithmic_bytes_per_launch": mix_bytes,
            "achieved": mix_bytes / (mix_ms * 1e-3) / 1e9, "frac": mix_bytes / (mix_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "same_stage_from_pytorch_ops_plus_btp_kernel_ms": unfused_ms, "speedup": unfused_ms / mix_ms,
            "backward": {
                "avg_launch_ms": mix_bwd_ms, "algorithmic_bytes_per_launch": mix_bwd_bytes,
                "achieved": mix_bwd_bytes / (mix_bwd_ms * 1e-3) / 1e9,
                "frac": mix_bwd_bytes / (mix_bwd_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            },
            "ceilings_GBps": {
                "what": "spear_btp_stream_probe_mix on the same buffers: no arithmetic / with a chain of dependent FMAs (640 forward, 1280 backward)",
                "forward_3_inputs_1_output": [ceil_fwd, ceil_fwd_c],
                "backward_4_inputs_3_outputs": [ceil_bwd, ceil_bwd_c],
            },
            "fwd_plus_bwd_ms": mix_ms + mix_bwd_ms,
            "same_stage_fwd_plus_bwd_from_pytorch_ops_plus_btp_kernels_ms": unfused_train_ms,
            "train_speedup": unfused_train_ms / (mix_ms + mix_bwd_ms),
            "qkv_gate_form": {
                "what": "out = q * btp(exp(gate), k * v) + v on [B, L, H, 16] bf16 with an fp32 log-decay gate; dq, dk, dv, dgate",
                "forward_ms": qkv_ms, "backward_ms": qkv_bwd_ms, "tokens_per_s": B * L / ((qkv_ms + qkv_bwd_ms) * 1e-3),
                "algorithmic_bytes_per_unit": {"forward": 132, "backward": 232},
                "achieved": (qkv_bytes + qkv_bwd_bytes) / ((qkv_ms + qkv_bwd_ms) * 1e-3) / 1e9,
                "frac": (qkv_bytes + qkv_bwd_bytes) / ((qkv_ms + qkv_bwd_ms) * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            },
        }
        del msets
        return fused

    fused = guarded(fused_leg) if (H % 4 == 0 and not args.no_fused) else None

    # the Phalanx layer end to end (five projections + mixing stage) on x[B, L, H*16], forward and
    # forward+backward, for the reference's PyTorch-ops method, its kernel method and the fused method
    def layer_leg():
        from spear_amd import Phalanx

        dim = H * 16
        gl = torch.Generator(device="cpu").manual_seed(seed + 13)
        xl = torch.randn(B, L, dim, generator=gl).to(torch.bfloat16).to(dev).requires_grad_(True)
        gout = torch.randn(B, L, dim, generator=gl).to(torch.bfloat16).to(dev)
        layer = {"shape": {"B": B, "L": L, "dim": dim}, "unit": "ms", "methods": {}}
        weights = None
        for method in ("pytorch", "default", "fused"):
            torch.manual_seed(seed)
            mod = Phalanx(dim=dim, length=L, method=method, dtype=torch.bfloat16).to(dev)
            if weights is None:
                weights = mod.state_dict()
            else:
                mod.load_state_dict(weights)

            def layer_fwd():
                with torch.no_grad():
                    mod(xl)

            def layer_train():
                mod.zero_grad(set_to_none=True)
                xl.grad = None
                mod(xl).backward(gout)

            def layer_ms(fn, n=20):
                for _ in range(4):
                    fn()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(n):
                    fn()
                e1.record(stream)
                torch.cuda.synchronize()
                return e0.elapsed_time(e1) / n

            layer["methods"][method] = {"forward": layer_ms(layer_fwd), "forward_backward": layer_ms(layer_train)}
            del mod
        del xl, gout
        torch.cuda.empty_cache()
        return layer

    layer = guarded(layer_leg) if (H % 4 == 0 and not args.no_layer) else None

    # streaming form: prompt prefill (recurrence + y*C+V + state hand-over) on the same tensors, and
    # the one-token decode step on [B, H, 16] operands with fp32 state
    def streaming_leg():
        st_h = torch.zeros(B, H, 16, device=dev)
        st_c = torch.zeros(B, H, 16, device=dev)
        st_r = torch.ones(B, H, device=dev)

        def prefill(s):
            rc = lib.spear_jagged_prefill(s["coeff"].data_ptr(), s["x"].data_ptr(), s["dy"].data_ptr(),
                                          s["dx"].data_ptr(), None, s["y"].data_ptr(), st_h.data_ptr(),
                                          st_r.data_ptr(), st_c.data_ptr(), B, H, 16, L, 16, 0, 0, 2, 2, 0, sp)
            assert rc == 0, lib.spear_btp_last_error()

        prefill_ms = kernel_ms(prefill)
        prefill_bytes = B * H * L * (2 + 3 * 32 + 32) + B * H * (2 * 64 + 4)

        g = torch.Generator(device="cpu").manual_seed(seed + 11)
        tok = [{
            "a": torch.sigmoid(torch.randn(B, H, generator=g)).to(torch.bfloat16).to(dev),
            "x": torch.randn(B, H, 16, generator=g).to(torch.bfloat16).to(dev),
            "c": torch.randn(B, H, 16, generator=g).to(torch.bfloat16).to(dev),
            "v": torch.randn(B, H, 16, generator=g).to(torch.bfloat16).to(dev),
            "y": torch.empty(B, H, 16, device=dev, dtype=torch.bfloat16),
        } for _ in range(16)]
        counter = [0]
        step_stream = [sp]  # the stream the step kernel is launched on (the capture stream while recording)

        def decode(s):
            i = counter[0]
            counter[0] = (i + 1) % 16
            rc = lib.spear_jagged_step(s["a"].data_ptr(), s["x"].data_ptr(), s["c"].data_ptr(), s["v"].data_ptr(),
                                       s["y"].data_ptr(), st_h.data_ptr(), st_r.data_ptr(), st_c.data_ptr(),
                                       st_h.data_ptr(), st_r.data_ptr(), st_c.data_ptr(), B, H, 16, int(i == 15),
                                       0, 0, 2, 2, 0, 0.0, step_stream[0])
            assert rc == 0, lib.spear_btp_last_error()

        def decode_torch(s):  # the same update as a chain of PyTorch ops (spear/nn/phalanx/inference.py:200-262)
            i = counter[0]
            counter[0] = (i + 1) % 16
            a = s["a"].unsqueeze(-1)
            h = a * st_h + s["x"]
            r = s["a"] * st_r
            s["y"].copy_((h + r.unsqueeze(-1) * st_c) * s["c"] + s["v"])
            if i == 15:
                st_c.copy_(h)
                st_h.zero_()
                st_r.fill_(1.0)
            else:
                st_h.copy_(h)
                st_r.copy_(r)

        def tokens_ms(fn):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            for i in range(16):
                fn(tok[i])
            torch.cuda.synchronize()
            n = 16 * max(4, args.steps // 16)
            e0.record(stream)
            for i in range(n):
                fn(tok[i % 16])
            e1.record(stream)
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / n

        step_ms, step_torch_ms = tokens_ms(decode), tokens_ms(decode_torch)

        # the same 16 launches of one block period as a HIP graph (no memset nodes: the step kernel
        # resets the state itself at the boundary)
        def period():
            for i in range(16):
                decode(tok[i])

        counter[0] = 0
        side = torch.cuda.Stream()
        side.wait_stream(stream)
        step_stream[0] = ctypes.c_void_p(side.cuda_stream)
        with torch.cuda.stream(side):
            period()  # warm-up on the capture stream
        stream.wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            period()
        step_stream[0] = sp
        torch.cuda.synchronize()
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        n_rep = max(4, args.steps // 16)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(n_rep):
            graph.replay()
        e1.record(stream)
        torch.cuda.synchronize()
        step_graph_ms = e0.elapsed_time(e1) / (16 * n_rep)
        # the whole layer for one token: four projections, the layer-layout step kernel (gates + state update +
        # y*C+V on the projections' [B, features] outputs, block position on the device), output projection;
        # eager and as ONE HIP graph replayed per token
        def layer_decode():
            from spear_amd import Phalanx
            from spear_amd.nn.phalanx.inference import PhalanxStepState, phalanx_step

            dim = H * 16
            torch.manual_seed(seed)
            mod = Phalanx(dim=dim, length=L, method="fused", dtype=torch.bfloat16).to(dev)
            gl = torch.Generator(device="cpu").manual_seed(seed + 17)
            xs = torch.randn(16, B, dim, generator=gl).to(torch.bfloat16).to(dev)
            st8 = PhalanxStepState.zeros(B, H, dev)
            y_buf = torch.empty(B, dim, device=dev, dtype=torch.bfloat16)
            x_buf = xs[0].clone()

            def timed(fn, n):
                for i in range(16):
                    fn(i)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for i in range(n):
                    fn(i)
                torch.cuda.synchronize()
                return (time.perf_counter() - t0) * 1e3 / n

            n_tok = 16 * max(4, args.steps // 16)
            eager_ms = timed(lambda i: phalanx_step(mod, xs[i % 16], st8, out=y_buf), n_tok)
            side2 = torch.cuda.Stream()
            side2.wait_stream(stream)
            with torch.cuda.stream(side2):
                phalanx_step(mod, x_buf, st8, out=y_buf)
            stream.wait_stream(side2)
            g2 = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g2, stream=side2):
                phalanx_step(mod, x_buf, st8, out=y_buf)
            torch.cuda.synchronize()
            graph_ms = timed(lambda i: g2.replay(), n_tok)

            def step_only(i):  # the mixing-stage kernel alone on precomputed projections
                _btp.mix_step(pa, pb, pc, pv, mixed, st8.h_loc, st8.r_pref, st8.c_prev_loc, st8.pos, False, 16, H, H)

            xc = xs[0]
            pa, pb, pc, pv = (q(xc) for q in (mod.param.proj_a, mod.param.proj_b, mod.param.proj_c, mod.param.proj_v))
            mixed = torch.empty_like(pv)
            kernel_ms_ = timed(step_only, n_tok)
            return {"what": "one token through the Phalanx layer at this batch: 4 projections + layer-layout step kernel + proj_out",
                    "eager_ms_per_token": eager_ms, "hip_graph_ms_per_token": graph_ms,
                    "tokens_per_s_graph": B / (graph_ms * 1e-3), "step_kernel_call_ms": kernel_ms_}

        layer_step = guarded(layer_decode) if H % 4 == 0 else None
        step_bytes = B * H * (2 + 8 + 3 * 32 + 32 + 2 * 64 + 64)  # a, r in/out, x c v, y, h in/out, c_prev
        streaming = {
            "prefill": {"avg_launch_ms": prefill_ms, "algorithmic_bytes_per_launch": prefill_bytes,
                        "achieved": prefill_bytes / (prefill_ms * 1e-3) / 1e9,
                        "frac": prefill_bytes / (prefill_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS},
            "decode_step": {"avg_launch_ms": step_ms, "algorithmic_bytes_per_launch": step_bytes,
                            "achieved": step_bytes / (step_ms * 1e-3) / 1e9,
                            "frac": step_bytes / (step_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                            "tokens_per_s": B / (step_ms * 1e-3),
                            "same_step_from_pytorch_ops_ms": step_torch_ms, "speedup": step_torch_ms / step_ms,
                            "avg_launch_ms_in_hip_graph": step_graph_ms},
            "layer_decode_step": layer_step,
        }
        return streaming

    streaming = None if args.no_streaming else guarded(streaming_leg)

    # The other full-size configurations (long rows: B=16 H=64 L=8192; log-space stress: B=64 H=128 L=2048; rows that
    # do not end on a cache line: B=64 H=128 L=2032; rows that do not fill whole spans: L=64 and L=192), each timed
    # in this same run: stand-alone forward, backward and forward+backward step, and the fused layer-layout
    # forward / backward on tensors of the same size. Three rotating buffer sets (2.3-12 GiB: nothing is served
    # from the 256 MiB memory-side cache), inputs drawn on the device with the configurations' distributions
    # (values do not change the time), HIP events on the launch stream.
    def other_config_leg(name, n_sets=3, n_steps=40):
        Bc, Hc, Lc, seed_c, x_std_c, gate_c = CONFIGS[name]
        gd = torch.Generator(device=dev).manual_seed(seed_c)
        Fc = Hc * 16

        def draw_gate():
            if gate_c == "sigmoid":
                return -torch.nn.functional.softplus(torch.randn(Bc, Hc, Lc, device=dev, generator=gd))
            forget = torch.rand(Bc, Hc, 1, device=dev, generator=gd) < 0.5
            lo = -20.0 + 15.0 * torch.rand(Bc, Hc, Lc, device=dev, generator=gd)
            hi = -1e-4 * torch.rand(Bc, Hc, Lc, device=dev, generator=gd)
            return torch.where(forget, lo, hi)

        def timed(fn, pool):
            for i in range(4):
                fn(pool[i % len(pool)])
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            for i in range(n_steps):
                fn(pool[i % len(pool)])
            e1.record(stream)
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / n_steps

        pool = []
        for _ in range(n_sets):
            pool.append({
                "coeff": torch.exp(draw_gate()).to(torch.bfloat16),
                "x": (torch.randn(Bc, Hc, 16, Lc, device=dev, generator=gd) * x_std_c).to(torch.bfloat16),
                "dy": torch.randn(Bc, Hc, 16, Lc, device=dev, generator=gd).to(torch.bfloat16),
                "y": torch.empty(Bc, Hc, 16, Lc, device=dev, dtype=torch.bfloat16),
                "dx": torch.empty(Bc, Hc, 16, Lc, device=dev, dtype=torch.bfloat16),
                "dA": torch.empty(Bc, Hc, Lc, device=dev, dtype=torch.float32),
            })

        def fwd_c(s):
            rc = lib.spear_btp_forward(s["coeff"].data_ptr(), s["x"].data_ptr(), s["y"].data_ptr(), None,
                                       Bc, Hc, Lc, 2, 0, 0, 0, sp)
            assert rc == 0, lib.spear_btp_last_error()

        def bwd_c(s):
            rc = lib.spear_btp_backward(s["coeff"].data_ptr(), s["x"].data_ptr(), s["dy"].data_ptr(), None,
                                        s["dx"].data_ptr(), s["dA"].data_ptr(), Bc, Hc, Lc, 2, 0, 0, 0, sp)
            assert rc == 0, lib.spear_btp_last_error()

        def step_c(s):
            fwd_c(s)
            bwd_c(s)

        units_c = Bc * Hc * Lc
        f_ms, b_ms, s_ms = timed(fwd_c, pool), timed(bwd_c, pool), timed(step_c, pool)
        frac = lambda nbytes_, ms: nbytes_ / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS
        res = {
            "workload": f"B={Bc} H={Hc} L={Lc} bf16, {n_sets} buffer sets, {n_steps} timed launches each",
            "forward_ms": f_ms, "forward_frac": frac(units_c * FWD_BYTES, f_ms),
            "backward_ms": b_ms, "backward_frac": frac(units_c * BWD_BYTES, b_ms),
            "step_ms": s_ms, "step_frac": frac(units_c * (FWD_BYTES + BWD_BYTES), s_ms),
            "tokens_per_s": Bc * Lc / (s_ms * 1e-3),
            "backward_traffic": profiled_traffic(name, "bwd_scan")[0],
        }
        del pool
        torch.cuda.empty_cache()

        if name in LAYER_LAYOUT_CONFIGS:
            mpool = []
            for _ in range(n_sets):
                m = {"a": torch.randn(Bc, Lc, Hc, device=dev, generator=gd).to(torch.bfloat16)}
                for k_ in ("b", "c", "v", "dout"):
                    m[k_] = torch.randn(Bc, Lc, Fc, device=dev, generator=gd).to(torch.bfloat16)
                for k_ in ("out", "db", "dc", "dv"):
                    m[k_] = torch.empty(Bc, Lc, Fc, device=dev, dtype=torch.bfloat16)
                m["da"] = torch.empty(Bc, Lc, Hc, device=dev, dtype=torch.bfloat16)
                mpool.append(m)

            def mix_c(s):
                rc = lib.spear_phalanx_mix_forward(s["a"].data_ptr(), s["b"].data_ptr(), s["c"].data_ptr(),
                                                   s["v"].data_ptr(), s["out"].data_ptr(), Bc, Lc, Hc, Hc, 0, 0, sp)
                assert rc == 0, lib.spear_btp_last_error()

            def mix_bwd_c(s):
                rc = lib.spear_phalanx_mix_backward(s["a"].data_ptr(), s["b"].data_ptr(), s["c"].data_ptr(),
                                                    s["v"].data_ptr(), s["dout"].data_ptr(), s["da"].data_ptr(),
                                                    s["db"].data_ptr(), s["dc"].data_ptr(), s["dv"].data_ptr(),
                                                    Bc, Lc, Hc, Hc, 0, 0, sp)
                assert rc == 0, lib.spear_btp_last_error()

            mf_ms, mb_ms = timed(mix_c, mpool), timed(mix_bwd_c, mpool)
            res["fused_forward_ms"], res["fused_forward_frac"] = mf_ms, frac(units_c * 130, mf_ms)
            res["fused_backward_ms"], res["fused_backward_frac"] = mb_ms, frac(units_c * 228, mb_ms)
            del mpool
            torch.cuda.empty_cache()
        return res

    other_configs = {"what": "the other full-size configurations in the same run: stand-alone kernels (66 + 102 B per "
                             "(token, head)) and the fused layer-layout kernels (130 + 228 B); fractions of 8 TB/s"}
    if not args.no_other_configs:
        for name in sorted(CONFIGS):
            if name != args.config:
                other_configs[name] = guarded(lambda name=name: other_config_leg(name))

    # what a caller of the public op gets: y = btp(coeff, x); y.backward(dy) through autograd, torch.library
    # dispatch and the compiled binding, eager (host-bound on small shapes) and as a HIP-graph replay of the
    # same two ops, at this shape and at the batch of configuration 1 (B = 8)
    def public_op_leg():
        from spear_amd.ops.btp import btp as btp_op

        def measure(bs):
            s = sets[0]
            c, xx, g = (s[k][:bs].contiguous() for k in ("coeff", "x", "dy"))
            ck = torch.empty(0, device=dev)
            y, dx = torch.empty_like(xx), torch.empty_like(xx)
            dA = torch.empty(bs, H, L, device=dev)

            def eager():
                cl, xl = c.detach().requires_grad_(True), xx.detach().requires_grad_(True)
                btp_op(cl, xl, 2, 32, torch.bfloat16).backward(g)

            def eager_forward():  # inference: no autograd node
                with torch.no_grad():
                    btp_op(c, xx, 2, 32, torch.bfloat16)

            def ops_only():  # the two custom ops on preallocated outputs (what a graph can hold)
                torch.ops.spear_btp.forward(c, xx, y, ck, 2, 32)
                torch.ops.spear_btp.backward(c, xx, g, ck, dx, dA, 2, 32)

            def timed(fn, n):
                for _ in range(5):
                    fn()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(n):
                    fn()
                torch.cuda.synchronize()
                return (time.perf_counter() - t0) * 1e3 / n

            n = max(20, args.steps // 2)
            eager_ms, ops_ms, eager_fwd_ms = timed(eager, n), timed(ops_only, n), timed(eager_forward, n)
            def fwd_op_only():
                torch.ops.spear_btp.forward(c, xx, y, ck, 2, 32)
            gside = torch.cuda.Stream()
            gside.wait_stream(stream)
            with torch.cuda.stream(gside):
                fwd_op_only()
            stream.wait_stream(gside)
            fgraph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(fgraph, stream=gside):
                fwd_op_only()
            torch.cuda.synchronize()
            fwd_graph_ms = timed(fgraph.replay, n)
            side = torch.cuda.Stream()
            side.wait_stream(stream)
            with torch.cuda.stream(side):
                ops_only()
            stream.wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                ops_only()
            torch.cuda.synchronize()
            graph_ms = timed(graph.replay, n)
            return {"B": bs, "eager_autograd_ms": eager_ms, "two_ops_preallocated_ms": ops_ms, "hip_graph_replay_ms": graph_ms,
                    "eager_over_graph": eager_ms / graph_ms, "two_ops_over_graph": ops_ms / graph_ms,
                    "forward_only": {"eager_no_grad_ms": eager_fwd_ms, "hip_graph_replay_ms": fwd_graph_ms,
                                     "eager_over_graph": eager_fwd_ms / fwd_graph_ms}}

        def measure_fused(bs):
            """phalanx_mix(a, b, c, v) + backward on [bs, L, features] tensors: eager through the autograd node compiled
            into the binding, the two custom ops on preallocated outputs, and a HIP-graph replay of those two ops."""
            from spear_amd import phalanx_mix
            import spear_amd.ops.btp.fused  # noqa: F401  (registers the custom ops)

            F = H * 16
            gq = torch.Generator(device=dev).manual_seed(seed + 23)
            a = torch.randn(bs, L, H, device=dev, generator=gq).to(torch.bfloat16)
            b, c, v, dout = (torch.randn(bs, L, F, device=dev, generator=gq).to(torch.bfloat16) for _ in range(4))
            out = torch.empty_like(v)
            grads = [torch.empty_like(t) for t in (a, b, c, v)]

            def eager():
                leaves = [t.detach().requires_grad_(True) for t in (a, b, c, v)]
                phalanx_mix(*leaves, heads=H, kv_heads=H).backward(dout)

            def eager_python_node():  # the torch.autograd.Function over the custom ops (what torch.compile traces)
                leaves = [t.detach().requires_grad_(True) for t in (a, b, c, v)]
                spear_amd.ops.btp.fused._PhalanxMix.apply(*leaves, H, H).backward(dout)

            def ops_only():
                torch.ops.spear_btp.mix_forward(a, b, c, v, out, H, H)
                torch.ops.spear_btp.mix_backward(a, b, c, v, dout, *grads, H, H)

            def timed(fn, n):
                for _ in range(5):
                    fn()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(n):
                    fn()
                torch.cuda.synchronize()
                return (time.perf_counter() - t0) * 1e3 / n

            n = max(20, args.steps // 2)
            eager_ms, ops_ms, python_node_ms = timed(eager, n), timed(ops_only, n), timed(eager_python_node, n)
            side = torch.cuda.Stream()
            side.wait_stream(stream)
            with torch.cuda.stream(side):
                ops_only()
            stream.wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                ops_only()
            torch.cuda.synchronize()
            graph_ms = timed(graph.replay, n)
            return {"B": bs, "eager_autograd_ms": eager_ms, "eager_autograd_python_node_ms": python_node_ms,
                    "two_ops_preallocated_ms": ops_ms, "hip_graph_replay_ms": graph_ms,
                    "eager_over_graph": eager_ms / graph_ms}

        return {"what": "btp(coeff, x, output_dtype=bf16) + backward through the public op (wall clock per fwd+bwd)",
                "this_shape": measure(B), "config1_batch": measure(min(B, 8)),
                "fused_op_config1_batch": guarded(lambda: measure_fused(min(B, 8)))}

    public_op = guarded(public_op_leg)

    traffic_bytes, traffic_source = profiled_traffic(args.config, "bwd_scan")

    units = B * H * L
    tokens = B * L
    bwd_gbps = units * BWD_BYTES / (bwd_ms * 1e-3) / 1e9
    fwd_gbps = units * FWD_BYTES / (fwd_ms * 1e-3) / 1e9
    step_gbps = units * (FWD_BYTES + BWD_BYTES) / (ms_per_step * 1e-3) / 1e9

    out = {
        "metric": "BTP fwd+bwd tokens/s (B1024 L128 D512 bf16); % of HBM roofline",
        "value": tokens / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "ms_per_step_device": ms_per_step_device,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"BTP forward+backward, B={B} H={H} L={L} head_dim=16 block_len=16 k=2, bf16 coeff/x/y/dy/dx, fp32 dA ({args.config})",
            "arithmetic": "fp32 recurrences on bf16 storage",
            "buffer_sets": len(sets),
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "btp_bwd_scan_kernel<Bf16> (bf16 dy)",
            "achieved": bwd_gbps,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": bwd_gbps / HBM_PEAK_GBPS,
            "traffic": traffic_bytes,
            "traffic_source": traffic_source,
            "avg_launch_ms": bwd_ms,
            "algorithmic_bytes_per_launch": units * BWD_BYTES,
        },
        "forward_kernel": {"avg_launch_ms": fwd_ms, "achieved": fwd_gbps, "frac": fwd_gbps / HBM_PEAK_GBPS,
                           "algorithmic_bytes_per_launch": units * FWD_BYTES},
        "forward_kernel_mfma_path": {"avg_launch_ms": fwd_mfma_ms,
                                     "achieved": units * FWD_BYTES / (fwd_mfma_ms * 1e-3) / 1e9,
                                     "frac": units * FWD_BYTES / (fwd_mfma_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS},
        "backward_kernel_mfma_path": {"avg_launch_ms": bwd_mfma_ms,
                                      "achieved": units * BWD_BYTES / (bwd_mfma_ms * 1e-3) / 1e9,
                                      "frac": units * BWD_BYTES / (bwd_mfma_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS},
        "op_default_dtypes_fp32_y_fp32_dy": {
            "forward_ms": fwd_f32_ms, "backward_ms": bwd_f32_ms,
            "algorithmic_bytes_per_unit": {"forward": 98, "backward": 134},
            "forward_frac": units * 98 / (fwd_f32_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "backward_frac": units * 134 / (bwd_f32_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "forward_ceiling_1_read_2_writes_GBps": ceil_1r2w,  # no arithmetic / 320 dependent FMAs
        },
        "log_gate_entry_points": {"forward_ms": fwd_log_ms, "backward_ms": bwd_log_ms,
                                  "achieved": units * (68 + 108) / ((fwd_log_ms + bwd_log_ms) * 1e-3) / 1e9,
                                  "algorithmic_bytes_per_unit": {"forward": 68, "backward": 108}},
        "fused_layer_stage": fused,
        "streaming": streaming,
        "phalanx_layer": layer,
        "fwd_plus_bwd": {"achieved": step_gbps, "frac": step_gbps / HBM_PEAK_GBPS,
                         "algorithmic_bytes_per_step": units * (FWD_BYTES + BWD_BYTES)},
        "step_spread": spread,
        "copy_kernel": {"avg_launch_ms": copy_ms, "achieved": 2 * nbytes / (copy_ms * 1e-3) / 1e9,
                        "bytes_moved": 2 * nbytes},
        "ceilings": {
            "what": "same 4 KiB-per-wavefront non-temporal access shape as the kernels, no arithmetic, same buffers",
            "nt_copy_1r1w": {"avg_launch_ms": probe_copy_ms, "achieved": ceil_copy, "unit": "GB/s"},
            "nt_2r1w": {"avg_launch_ms": probe_2r1w_ms, "achieved": ceil_2r1w, "unit": "GB/s"},
            "forward_kernel_vs_nt_copy": fwd_gbps / ceil_copy,
            "backward_kernel_vs_nt_2r1w": bwd_gbps / ceil_2r1w,
            "other_launch_shapes_GBps": probe_shapes,
            "forward_kernel_vs_best_copy_shape": fwd_gbps / best_copy,
            "backward_kernel_vs_best_2r1w_shape": bwd_gbps / best_2r1w,
            "read_only_GBps": read_rate, "write_only_GBps": write_rate,
            "nt_2r1w_with_640_dependent_fma_GBps": with_compute_2r1w,
            "backward_kernel_vs_2r1w_with_compute": bwd_gbps / with_compute_2r1w,
            "serial_read_plus_write_model": {
                "what": "algorithmic GB/s if a kernel's reads and writes run one after the other at the two rates above",
                "forward_34R_32W": floor_fwd, "backward_66R_36W": floor_bwd,
                "forward_kernel_vs_model": fwd_gbps / floor_fwd, "backward_kernel_vs_model": bwd_gbps / floor_bwd,
                "fused_forward_98R_32W": serial_floor(98, 32), "fused_backward_130R_98W": serial_floor(130, 98),
            },
        },
        "public_op": public_op,
        "other_configs": other_configs,
    }
    if not args.no_cpu_baseline:
        base = cpu_baseline(B, H, L, seed, x_std, gate)
        out["cpu_baseline"] = base
        out["speedup_vs_cpu_baseline"] = out["value"] / base["value"]
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
