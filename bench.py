#!/usr/bin/env python3
"""Benchmark of the memory-saving correlation separation on one MI355X.

A step is one pass of the hot path over one synthetic batch, called through the C ABI with every
input already resident in HBM: max/argmax/avg forward, attention-compression forward, compression
backward, max/avg backward (the default workload, benchmark configuration 4: B=2, C=256, 55x128, K'=4).
Prints ONE JSON line.  `value` is algorithmic TFLOP/s: (contraction passes x 2*B*N1*N2*C) / time,
with passes = 7 for forward+backward with attention; epilogue flops are not counted.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # 256 CU x 256 flop/clk x 2.4 GHz
METRIC = "fused corr-separation fwd+bwd ms and MFMA TFLOP/s at B=2, C=256, 55×128"

# name -> (B, H, W, K', ops).  ops: f = max/avg(+argmax) fwd, c = compression fwd, C = compression bwd, F = max/avg bwd
WORKLOADS = {
    "cfg1": (1, 48, 64, 0, "f"),
    "cfg2": (4, 48, 64, 0, "fF"),
    "cfg3": (1, 55, 128, 4, "fc"),
    "cfg4": (2, 55, 128, 4, "fcCF"),
    "cfg5": (1, 136, 240, 4, "fc"),
}
PASSES = {"f": 1, "c": 1, "C": 3, "F": 2}
# contraction passes (units of W = 2*B*N1*N2*C flops) executed by one launch of each kernel
KERNEL_PASSES = {"df1_both": 1, "df2_both": 1, "fwd_maxavg": 1, "fwd_weighted": 1, "df1_comp": 1, "df2_comp": 1, "df1_maxavg": 1, "df2_maxavg": 1}
# HBM bytes per launch at cfg4 from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs, scaled by the factors a
# 256 MiB device copy gives in the same run (profiles/cfg4_fwd_bwd_kernels.txt); None = not measured
_MIB = 2 ** 20
TRAFFIC_BYTES_CFG4 = {"fwd_maxavg": 115.9 * _MIB, "fwd_weighted": 187.6 * _MIB, "df1_comp": 202.6 * _MIB,
                      "df2_comp": 289.1 * _MIB, "df1_maxavg": 153.4 * _MIB, "df2_maxavg": 203.7 * _MIB,
                      "df1_both": 232.1 * _MIB, "df2_both": 438.6 * _MIB}


def make_inputs(B, H, W, C, Kp, torch):
    """Seeded CPU tensors exactly as the caller builds them (core/corr.py:419-422)."""
    g = torch.Generator().manual_seed(1234)
    fmap1 = torch.randn(B, C, H, W, generator=g)
    fmap2 = torch.randn(B, C, H, W, generator=g)
    f1 = fmap1.permute(0, 2, 3, 1).contiguous() / torch.sqrt(torch.tensor(C).float())
    f2 = fmap2.permute(0, 2, 3, 1).contiguous()
    grads = dict(g_u=torch.randn(B, H, W, 2, H, generator=g), g_v=torch.randn(B, H, W, 2, W, generator=g))
    if Kp:
        grads.update(g_cu=torch.randn(B, H, W, Kp, H, generator=g), g_cv=torch.randn(B, H, W, Kp, W, generator=g))
    torch.manual_seed(1234)
    att = (torch.nn.Conv3d(2, Kp, 3, padding=1), torch.nn.Conv3d(2, Kp, 3, padding=1)) if Kp else None
    return f1, f2, grads, att


def cpu_baseline(B, H, W, C, Kp, ops, torch, budget_s=20.0):
    """The full-4D PyTorch path (oracle restatement of core/corr.py) timed on the host cores.

    Bounded sample: batch 1 of the workload, repeated until ~budget_s of CPU time is spent.
    """
    from oracle import oracle as O
    f1, f2, grads, att = make_inputs(1, H, W, C, Kp, torch)
    backward = "C" in ops or "F" in ops
    threads = torch.get_num_threads()

    def once():
        x1 = f1.clone().requires_grad_(backward)
        x2 = f2.clone().requires_grad_(backward)
        with torch.set_grad_enabled(backward):
            s = O.corr_volume(x1, x2)
            out_u = torch.stack((s.max(dim=4)[0], s.mean(dim=4)), dim=3)
            out_v = torch.stack((s.max(dim=3)[0], s.mean(dim=3)), dim=3)
            loss = (out_u * grads["g_u"]).sum() + (out_v * grads["g_v"]).sum() if backward else None
            if Kp:
                a_u = att[0](out_v.permute(0, 3, 4, 1, 2)).softmax(dim=2).permute(0, 3, 4, 1, 2)
                a_v = att[1](out_u.permute(0, 3, 4, 1, 2)).softmax(dim=2).permute(0, 3, 4, 1, 2)
                cu, cv = O.compression_from_volume(s, a_u, a_v)
                if backward:
                    loss = loss + (cu * grads["g_cu"]).sum() + (cv * grads["g_cv"]).sum()
            if backward:
                loss.backward()

    once()  # warm-up (allocator, thread pool)
    n, t0 = 0, time.perf_counter()
    while True:
        once()
        n += 1
        dt = time.perf_counter() - t0
        if dt >= budget_s or n >= 20:
            break
    ms = dt / n * 1e3
    passes = sum(PASSES[o] for o in ops)
    flops = passes * 2.0 * 1 * (H * W) ** 2 * C
    return {
        "value": round(flops / (ms * 1e-3) / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "ms_per_step": round(ms, 1),
        "sample": f"batch 1 of the workload (B=1, {H}x{W}, C={C}, K'={Kp}), full-4D torch path "
                  f"{'fwd+bwd via autograd' if backward else 'fwd'}, {n} repeats after 1 warm-up, same algorithmic flop count",
    }


def module_level(B, H, W, C, Kp, torch, dev, reps=5):
    """The caller's whole separate() over 4 pyramid levels through the drop-in classes (untimed extra):
    NHWC copies, both operators per level, the fused attention producer and volume assembly, autograd."""
    from separableflowthesis_amd import AlternateCorrBlockSepflow
    g = torch.Generator().manual_seed(1234)
    fmap1 = torch.randn(B, C, H, W, generator=g).to(dev).requires_grad_()
    fmap2 = torch.randn(B, C, H, W, generator=g).to(dev).requires_grad_()
    torch.manual_seed(1234)
    att = tuple(torch.nn.Conv3d(2, Kp, 3, padding=1).to(dev) for _ in range(2)) if Kp else None

    def run(backward):
        blk = AlternateCorrBlockSepflow(fmap1, fmap2, None, 4, 4, support_backward=backward)
        c1, c2 = blk(None, sep=True, attention_weights=att)
        if backward:
            (c1.sum() + c2.sum()).backward()

    out = {}
    for name, bw in (("forward_ms", False), ("forward_backward_ms", True)):
        for _ in range(2):
            run(bw)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(reps):
            run(bw)
        torch.cuda.synchronize()
        out[name] = round((time.perf_counter() - t0) / reps * 1e3, 3)
    out["what"] = f"AlternateCorrBlockSepflow.separate, 4 levels, B={B}, C={C}, {H}x{W}, K'={Kp}, torch autograd around the native ops"
    return out


def lookup_level(B, H, W, C, torch, dev, reps=20):
    """corr_fn(coords) of the block without the 4D volume (untimed extra): 4 levels, radius 4, a smooth flow field.
    Forward = one gather kernel; backward = grid gradients, d_f1 gather, d_f2 by owner tiles, slice reduction."""
    from separableflowthesis_amd import MemorySaver
    g = torch.Generator().manual_seed(1234)
    f1 = torch.randn(B, H, W, C, generator=g).to(dev)
    f2s = [torch.randn(B, H >> l, W >> l, C, generator=g).to(dev) for l in range(4)]
    yy, xx = torch.meshgrid(torch.arange(H), torch.arange(W), indexing="ij")
    flow = torch.randn(B, 2, 1, 1, generator=g) * 4 + torch.randn(B, 2, H, W, generator=g) * 0.5
    coords = (torch.stack([xx, yy]).float()[None] + flow).contiguous().to(dev)
    up = torch.randn(B, 4 * 81, H, W, generator=g).to(dev)
    scale = 1.0 / 16.0

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps

    fwd = timed(lambda: MemorySaver.lookup_forward(f1, f2s, coords, 4, scale))
    bwd = timed(lambda: MemorySaver.lookup_backward(f1, f2s, coords, up, 4, scale))
    # the lookup in the two separated volumes (CorrBlock1D): one aggregated channel as in the model, and all 24
    one_d = {}
    for dim in (1, 24):
        c1 = torch.randn(B, dim, W, H, W, generator=g).to(dev)
        c2 = torch.randn(B, dim, H, H, W, generator=g).to(dev)
        u = torch.randn(B, 4 * dim * 9, H, W, generator=g).to(dev)

        def f1d():
            MemorySaver.lookup1d_forward(c1, coords, 0, True, 4, 4)
            MemorySaver.lookup1d_forward(c2, coords, 1, False, 4, 4)

        def b1d():
            MemorySaver.lookup1d_backward(coords, u, tuple(c1.shape), 0, True, 4, 4)
            MemorySaver.lookup1d_backward(coords, u, tuple(c2.shape), 1, False, 4, 4)

        one_d[f"dim{dim}"] = {"forward_ms": round(timed(f1d), 4), "backward_ms": round(timed(b1d), 4),
                              "volumes_mib": round((c1.numel() + c2.numel()) * 4 / 2 ** 20, 1)}
        del c1, c2, u
    pts = B * H * W * 4 * 100                       # (pixel, level, grid point) pairs: one C-long dot product each
    alg = (f1.numel() + sum(t.numel() for t in f2s) + coords.numel() + up.numel()) * 4   # up has the output's size
    return {
        "forward_ms": round(fwd, 4), "backward_ms": round(bwd, 4),
        "forward_window_gb_s": round(pts * C * 4 / fwd / 1e6, 1),
        "forward_gflop_s": round(pts * C * 2 / fwd / 1e6, 1),
        "forward_algorithmic_mib": round(alg / 2 ** 20, 1),
        "forward_hbm_gb_s": round(alg / fwd / 1e6, 1),
        "volumes_1d": one_d,
        "what": f"sepcorr_lookup_forward / sepcorr_lookup_backward, B={B}, C={C}, {H}x{W}, 4 levels, radius 4; "
                "window = bytes of the fmap2 rows under all windows (one C-long dot product each, 2 flop per 4 bytes; "
                "the kernel fetches a row once for four neighbouring pixels, so this may exceed the vector cache's "
                "256 CU x 64 B/clk x 2.4 GHz = 39.3 TB/s); algorithmic = f1 + pyramid + coords + out once; "
                "volumes_1d = CorrBlock1D on both separated volumes (sepcorr_lookup1d_forward/backward, 4 levels, radius 4)",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="cfg4", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--profile-steps", type=int, default=5)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three 256 MiB device copies (known traffic) for scaling rocprofv3 FETCH_SIZE/WRITE_SIZE")
    ap.add_argument("--module-level", action="store_true",
                    help="measure the caller's whole separate() too even with --no-cpu-baseline")
    ap.add_argument("--only-module-level", action="store_true",
                    help="measure nothing but the caller's whole separate() (for kernel traces of that path)")
    ap.add_argument("--only-lookup", action="store_true", help="run only the pyramid-lookup extra (for profiling)")
    ap.add_argument("--single-stream", action="store_true",
                    help="keep all kernels of a call on the caller's stream (per-kernel durations under a profiler are "
                         "then those of kernels running alone)")
    args = ap.parse_args()
    if args.single_stream:
        os.environ["SEPCORR_SINGLE_STREAM"] = "1"
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1")

    import torch
    from separableflowthesis_amd import _lib
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    B, H, W, Kp, ops = WORKLOADS[args.workload]
    C = 256
    N = H * W
    if args.only_lookup:
        print(json.dumps({"workload": args.workload, "lookup": lookup_level(B, H, W, C, torch, dev)}))
        return
    if args.only_module_level:
        print(json.dumps({"workload": args.workload, "module_level": module_level(B, H, W, C, Kp, torch, dev)}))
        return
    f1c, f2c, gr, att = make_inputs(B, H, W, C, Kp, torch)
    f1, f2 = f1c.to(dev), f2c.to(dev)
    gr = {k: v.to(dev) for k, v in gr.items()}
    E = lambda *s, dt=torch.float32: torch.empty(*s, dtype=dt, device=dev)
    out_u, out_v = E(B, H, W, 2, H), E(B, H, W, 2, W)
    am_u, am_v = E(B, H, W, 1, H, dt=torch.int32), E(B, H, W, 1, W, dt=torch.int32)
    d1, d2, d1b, d2b = E(B, H, W, C), E(B, H, W, C), E(B, H, W, C), E(B, H, W, C)
    nws = lib.sepcorr_backward_workspace_bytes(B, H, W, H, W, C)
    ws = torch.empty(max(nws, 256), dtype=torch.uint8, device=dev)
    dims = (B, H, W, H, W, C)
    stream = torch.cuda.current_stream().cuda_stream
    P = lambda t: t.data_ptr()

    def op_f():
        _lib.check(lib.sepcorr_max_argmax_avg_forward(P(f1), P(f2), P(out_u), P(out_v), P(am_u), P(am_v), *dims, stream))

    op_f()
    if Kp:
        # attention weights as the caller produces them: Conv3d on the (max,avg) volumes, softmax over the
        # kept axis, back to (B,H1,W1,K',L) (core/corr.py:437-446)
        from separableflowthesis_amd import MemorySaver
        with torch.no_grad():
            a_u = MemorySaver.attention_forward(out_v, att[0].weight.to(dev).contiguous(), att[0].bias.to(dev))
            a_v = MemorySaver.attention_forward(out_u, att[1].weight.to(dev).contiguous(), att[1].bias.to(dev))
        cu, cv = E(B, H, W, Kp, H), E(B, H, W, Kp, W)
        da_u, da_v = torch.empty_like(a_u), torch.empty_like(a_v)

    def op_c():
        _lib.check(lib.sepcorr_compression_forward(P(f1), P(f2), P(a_u), P(a_v), P(cu), P(cv), *dims, Kp, stream))

    def op_C():
        _lib.check(lib.sepcorr_compression_backward(P(f1), P(f2), P(a_u), P(a_v), P(gr["g_cu"]), P(gr["g_cv"]),
                                                    P(d1), P(d2), P(da_u), P(da_v), *dims, Kp, P(ws), nws, stream))

    def op_F():
        _lib.check(lib.sepcorr_max_argmax_avg_backward(P(f1), P(f2), P(am_u), P(am_v), P(gr["g_u"]), P(gr["g_v"]),
                                                       P(d1b), P(d2b), *dims, P(ws), nws, stream))

    table = {"f": op_f, "c": op_c, "C": op_C, "F": op_F}
    seq = [table[o] for o in ops]

    def step():
        for fn in seq:
            fn()

    if args.calibrate_copy:
        src = torch.empty(64 * 2**20, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    torch.cuda.reset_peak_memory_stats()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3

    # per-kernel durations: HIP events recorded by the library on the launch stream
    lib.sepcorr_profile_enable(1)
    for _ in range(max(1, args.profile_steps)):
        step()
    torch.cuda.synchronize()
    cap = 4096
    names = ctypes.create_string_buffer(1 << 16)
    tms = (ctypes.c_float * cap)()
    n = lib.sepcorr_profile_collect(names, len(names), tms, cap)
    lib.sepcorr_profile_enable(0)
    per = {}
    for nm, t in zip(names.value.decode().split("\n")[:n], list(tms)[:n]):
        per.setdefault(nm, []).append(t)
    Wf = 2.0 * B * N * N * C
    kernels = {}
    for nm, ts in per.items():
        avg = sum(ts) / len(ts)
        calls = len(ts) / max(1, args.profile_steps)
        ent = {"avg_ms": round(avg, 4), "launches_per_step": round(calls, 2)}
        if nm in KERNEL_PASSES:
            ent["tflops"] = round(KERNEL_PASSES[nm] * Wf / (avg * 1e-3) / 1e12, 2)
        kernels[nm] = ent
    dom = max((k for k in kernels if k in KERNEL_PASSES),
              key=lambda k: kernels[k]["avg_ms"] * kernels[k]["launches_per_step"])
    ach = kernels[dom]["tflops"]
    passes = sum(PASSES[o] for o in ops)
    value = passes * Wf / (ms * 1e-3) / 1e12

    out = {
        "metric": METRIC, "value": round(value, 3), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{args.workload}: B={B}, C={C}, {H}x{W}, K'={Kp}, ops={ops} "
                               "(f=max/argmax/avg fwd, c=compression fwd, C=compression bwd, F=max/avg bwd)",
                   "contraction_passes": passes, "gflop_per_step": round(passes * Wf / 1e9, 2),
                   "frac_of_fp32_mfma_peak": round(value / PEAK_FP32_MFMA_TFLOPS, 4),
                   "peak_hbm_allocated_mib": round(torch.cuda.max_memory_allocated() / 2**20, 1),
                   "volume_4d_never_allocated_mib": round(B * N * N * 4 / 2**20, 1)},
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": ach, "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(ach / PEAK_FP32_MFMA_TFLOPS, 4), "traffic": TRAFFIC_BYTES_CFG4.get(dom) if args.workload == "cfg4" else None},
        "kernels": kernels,
    }
    fused_step = None
    if "C" in ops and "F" in ops:
        # The same job through the entry points that have no counterpart in the reference's two-operator API:
        # weight gradients alone, then one contraction per feature gradient with dL/dS of both operators added
        # (5 sweeps over the volume instead of 7).  Reported beside the headline, never as `value`.
        def fused_step():
            op_f()
            op_c()
            _lib.check(lib.sepcorr_compression_backward(P(f1), P(f2), P(a_u), P(a_v), P(gr["g_cu"]), P(gr["g_cv"]),
                                                        None, None, P(da_u), P(da_v), *dims, Kp, None, 0, stream))
            _lib.check(lib.sepcorr_fused_backward(P(f1), P(f2), P(am_u), P(am_v), P(gr["g_u"]), P(gr["g_v"]),
                                                  P(a_u), P(a_v), P(gr["g_cu"]), P(gr["g_cv"]), P(d1), P(d2),
                                                  *dims, Kp, P(ws), nws, stream))
        for _ in range(args.warmup):
            fused_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            fused_step()
        torch.cuda.synchronize()
        fms = (time.perf_counter() - t0) / args.steps * 1e3
        out["fused_level"] = {
            "ms_per_step": round(fms, 4), "contraction_passes_executed": 5,
            "tflops_executed": round(5 * Wf / (fms * 1e-3) / 1e12, 2),
            "what": "same inputs and outputs as the headline step (d_f1, d_f2 are the sums of the two operators' "
                    "gradients), via sepcorr_compression_backward(d_f1=d_f2=NULL) + sepcorr_fused_backward"}
    # The same headline step with the forward sweeps contracting in three bf16 planes per operand (an option of
    # this library with the same accuracy bar, see sepcorr_set_contraction).  Reported beside the headline, never
    # as `value`: the headline arithmetic is fp32 MFMA throughout.
    prev_mode = lib.sepcorr_set_contraction(1)
    try:
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        pms = (time.perf_counter() - t0) / args.steps * 1e3
        lib.sepcorr_profile_enable(1)
        step()
        torch.cuda.synchronize()
        names = ctypes.create_string_buffer(1 << 16)
        tms = (ctypes.c_float * 4096)()
        n = lib.sepcorr_profile_collect(names, len(names), tms, 4096)
        lib.sepcorr_profile_enable(0)
        pk = {}
        for nm, t in zip(names.value.decode().split("\n")[:n], list(tms)[:n]):
            if nm.endswith("bf16x3") or nm.startswith("split_planes") or nm == "df1_reduce_chunks":
                pk.setdefault(nm, []).append(t)
        out["bf16_planes"] = {
            "ms_per_step": round(pms, 4), "tflops_fp32_equivalent": round(passes * Wf / (pms * 1e-3) / 1e12, 2),
            "kernels_ms": {k: round(sum(v) / len(v), 4) for k, v in pk.items()},
            "what": "headline step with sepcorr_set_contraction(SEPCORR_CONTRACT_BF16X3): forward-type sweeps "
                    "(max/argmax/avg, compression forward, attention gradients) and d_f1 in bf16 planes, d_f2 "
                    "in fp32 MFMA"}
        if fused_step is not None:
            for _ in range(args.warmup):
                fused_step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                fused_step()
            torch.cuda.synchronize()
            out["bf16_planes"]["fused_level_ms_per_step"] = round((time.perf_counter() - t0) / args.steps * 1e3, 4)
        if not args.no_cpu_baseline or args.module_level:
            ml = module_level(B, H, W, C, Kp, torch, dev)
            out["bf16_planes"]["module_level"] = {k: v for k, v in ml.items() if k != "what"}
    finally:
        lib.sepcorr_set_contraction(prev_mode)
    if not args.no_cpu_baseline or args.module_level:
        out["module_level"] = module_level(B, H, W, C, Kp, torch, dev)
    if not args.no_cpu_baseline or args.module_level:
        out["lookup"] = lookup_level(B, H, W, C, torch, dev)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(B, H, W, C, Kp, ops, torch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
