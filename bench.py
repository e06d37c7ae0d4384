#!/usr/bin/env python3
"""Benchmark of the memory-saving correlation separation on one MI355X.

A step is one pass of the hot path over one synthetic batch, called through the C ABI with every
input already resident in HBM.  The headline workload is benchmark configuration 4 (B=2, C=256, 55x128,
K'=4): max/argmax/avg forward, attention-compression forward, compression backward, max/avg backward.
Prints ONE JSON line.  `value` is the MFMA TFLOP/s of the step: (contraction passes executed on the matrix cores x
2*B*N1*N2*C) / time; epilogue flops are not counted.  The reference's formulation has 7 passes for forward+backward
with attention; where the library runs the max/avg backward as gathers instead of its two contractions, 5 of them
are executed and counted, and the algorithmic figure (7 passes over the same time) and the timing of the all-dense
step stand beside it (`algorithmic_tflops`, `all_dense`).  `ms_per_step` is the figure to compare builds by.  The same line
carries a `configs` table with all five benchmark configurations (ms/step, TFLOP/s, fraction of the
fp32 MFMA peak, peak HBM allocated, dominant-kernel roofline), the CPU baseline (full-4D torch path on
the host cores, one thread and all threads) and, as extras, the caller-level measurements.
"""
import argparse
import ctypes
import gc
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # 256 CU x 256 flop/clk x 2.4 GHz
METRIC = "fused corr-separation fwd+bwd ms and MFMA TFLOP/s at B=2, C=256, 55×128"
C = 256

# name -> (B, H, W, K', ops).  ops: f = max/avg(+argmax) fwd, c = compression fwd, C = compression bwd, F = max/avg bwd
WORKLOADS = {
    "cfg1": (1, 48, 64, 0, "f"),
    "cfg2": (4, 48, 64, 0, "fF"),
    "cfg3": (1, 55, 128, 4, "fc"),
    "cfg4": (2, 55, 128, 4, "fcCF"),
    "cfg5": (1, 136, 240, 4, "fc"),
}
OPS_TEXT = "(f=max/argmax/avg fwd, c=compression fwd, C=compression bwd, F=max/avg bwd)"
PASSES = {"f": 1, "c": 1, "C": 3, "F": 2}
# kernels that execute one contraction pass (W = 2*B*N1*N2*C flops) per launch
SWEEP_KERNELS = ("fwd_maxavg", "fwd_weighted", "df1_comp", "df2_comp", "df1_maxavg", "df2_maxavg", "df1_both", "df2_both")
_MIB = 2 ** 20


def measured_traffic(workload):
    """HBM bytes per launch by kernel label, from the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary committed
    under profiles/ for this workload (scaled there by what a plain copy of known size reads on the same
    counters).  Lines of the form `traffic <label> <fetch_KiB> <write_KiB> <MiB>`; {} when there is no summary."""
    path = os.path.join(ROOT, "profiles", f"{workload}_fwd_bwd_kernels.txt")
    out = {}
    if os.path.exists(path):
        for line in open(path):
            m = re.match(r"traffic\s+(\S+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s*$", line)
            if m:
                out[m.group(1)] = float(m.group(4)) * _MIB
        return out
    # the other configurations share one summary: `traffic <workload> <label> <fetch_KiB> <write_KiB> <MiB>`
    for path in sorted(os.listdir(os.path.join(ROOT, "profiles"))):
        for line in open(os.path.join(ROOT, "profiles", path)):
            m = re.match(r"traffic\s+(\S+)\s+(\S+)\s+([\d.]+)\s+([\d.]+)\s+([\d.]+)\s*$", line)
            if m and m.group(1) == workload:
                out[m.group(2)] = float(m.group(5)) * _MIB
    return out


def algorithmic_bytes(label, B, N, H, W, Kp):
    """Bytes a launch must move at least: every input read once, every output written once (fp32/int32)."""
    feat = B * N * C
    per_p_u, per_p_v = B * N * H, B * N * W          # one channel of a *_u / *_v tensor
    if label == "fwd_maxavg":
        n = 2 * feat + 3 * (per_p_u + per_p_v)         # f1, f2; max, avg, argmax of both volumes
    elif label == "fwd_weighted":
        n = 2 * feat + 2 * Kp * (per_p_u + per_p_v)    # f1, f2; K' weights in, K' sums out, both volumes
    else:
        fields = {"maxavg": 3, "comp": 2 * Kp, "both": 3 + 2 * Kp}[label.split("_")[1]]
        n = 2 * feat + fields * (per_p_u + per_p_v)    # one fmap in, one gradient out, the weight fields of dL/dS
    return 4 * n


def make_inputs(B, H, W, Kp, torch):
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


# ------------------------------------------------------------------------------------------------
# CPU baseline: the full-4D PyTorch path (oracle restatement of core/corr.py) on the host cores
# ------------------------------------------------------------------------------------------------

def _cpu_step(name, torch, pixel_fraction=1):
    """One step of workload `name` at batch 1 on the CPU; `pixel_fraction` > 1 keeps every n-th image-1 pixel row
    (image-1 pixels are independent units of the operator).  Returns a callable and the flops it stands for."""
    from oracle import oracle as O
    _, H, W, Kp, ops = WORKLOADS[name]
    f1, f2, grads, att = make_inputs(1, H, W, Kp, torch)
    if pixel_fraction > 1:
        rows = slice(0, H, pixel_fraction)
        f1 = f1[:, rows].contiguous()
        grads = {k: v[:, rows].contiguous() for k, v in grads.items()}
    backward = "C" in ops or "F" in ops
    n1 = f1.shape[1] * f1.shape[2]

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

    return once, sum(PASSES[o] for o in ops) * 2.0 * n1 * (H * W) * C


def _time_cpu(fn, budget_s, max_reps, min_reps=3):
    """Mean of at least `min_reps` repeats after one warm-up call; more while the time budget lasts."""
    fn()
    n, t0 = 0, time.perf_counter()
    while True:
        fn()
        n += 1
        dt = time.perf_counter() - t0
        if n >= min_reps and (dt >= budget_s or n >= max_reps):
            return dt / n * 1e3, n


def cpu_baseline(torch, headline="cfg4"):
    """Bounded sample of every workload at batch 1, each figure the mean of at least 3 repeats after a warm-up call:
    the headline with all host threads (~8 s) and with one thread, the other configurations with all threads;
    config 5 on every 8th image-1 pixel row (its whole 4D volume is 4.26 GB per copy)."""
    threads = torch.get_num_threads()
    fn, flops = _cpu_step(headline, torch)
    ms_all, n_all = _time_cpu(fn, 8.0, 12)
    torch.set_num_threads(1)
    try:
        ms_one, n_one = _time_cpu(fn, 0.0, 3)
    finally:
        torch.set_num_threads(threads)
    _, H, W, Kp, ops = WORKLOADS[headline]
    out = {
        "value": round(flops / (ms_all * 1e-3) / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "ms_per_step": round(ms_all, 1),
        "one_thread": {"value": round(flops / (ms_one * 1e-3) / 1e12, 4), "ms_per_step": round(ms_one, 1), "cores": 1},
        "host_cpus": os.cpu_count(),
        "sample": f"batch 1 of the workload (B=1, {H}x{W}, C={C}, K'={Kp}), full-4D torch path "
                  f"{'fwd+bwd via autograd' if 'C' in ops or 'F' in ops else 'fwd'}: {n_all} repeats after 1 warm-up with "
                  f"{threads} threads, {n_one} repeats after 1 warm-up with 1 thread; the other configurations 3 repeats "
                  f"after 1 warm-up each; same algorithmic flop count as the GPU step",
        "configs": {},
    }
    for name in sorted(WORKLOADS):
        if name == headline:
            out["configs"][name] = {"ms_per_step_b1": round(ms_all, 1), "tflops": out["value"], "cores": threads}
            continue
        frac = 8 if name == "cfg5" else 1
        fn, fl = _cpu_step(name, torch, frac)
        ms, nrep = _time_cpu(fn, 0.0, 3)
        ent = {"ms_per_step_b1": round(ms * frac, 1), "tflops": round(fl / (ms * 1e-3) / 1e12, 4), "cores": threads,
               "repeats": nrep}
        if frac > 1:
            ent["sample"] = f"every {frac}th image-1 pixel row, time scaled by {frac}"
        out["configs"][name] = ent
    return out


def stored_volume_path_memory(torch, dev, names=("cfg3", "cfg4", "cfg5")):
    """Part of the baseline leg: peak device memory of the stored-volume path (the oracle's CorrBlock4D: full 4D
    volume, pooled pyramid, max / mean / einsum / Conv3d / interpolate through torch autograd) run on the GPU in fp32
    at whole-batch size, forward and forward + backward (configuration 5 forward only), measured as the block's own
    figures are: peak of torch's allocator above what is held before the call, dense upstream gradients.  This is the
    second column of the both-models memory table of scripts/test_model.py:320-382."""
    from oracle import oracle as O
    out = {}
    for name in names:
        B, H, W, Kp, _ = WORKLOADS[name]
        g = torch.Generator().manual_seed(1234)
        fmap1 = torch.randn(B, C, H, W, generator=g).to(dev).requires_grad_()
        fmap2 = torch.randn(B, C, H, W, generator=g).to(dev).requires_grad_()
        torch.manual_seed(1234)
        att = tuple(torch.nn.Conv3d(2, Kp, 3, padding=1).to(dev) for _ in range(2))
        ups = None
        ent = {}
        for key, bw in (("forward", False), ("forward_backward", True)):
            if bw and name == "cfg5":
                continue
            gc.collect()
            torch.cuda.empty_cache()
            torch.cuda.synchronize()
            torch.cuda.reset_peak_memory_stats()
            base = torch.cuda.memory_allocated()
            with torch.set_grad_enabled(bw):
                c1, c2 = O.CorrBlock4D(fmap1, fmap2, num_levels=4).separate(att)
                if bw:
                    if ups is None:
                        ups = [torch.randn(c.shape, generator=g).to(dev) for c in (c1, c2)]
                        base += sum(u.numel() * 4 for u in ups)   # held by the layers above, as in module_level()
                    torch.autograd.backward([c1, c2], ups)
            torch.cuda.synchronize()
            ent[f"stored_4d_path_{key}_peak_allocated_mib"] = round((torch.cuda.max_memory_allocated() - base) / _MIB, 1)
            del c1, c2
        out[name] = ent
        del fmap1, fmap2, att, ups
        gc.collect()
        torch.cuda.empty_cache()
    return out


# ------------------------------------------------------------------------------------------------
# GPU: one workload through the C ABI
# ------------------------------------------------------------------------------------------------

class Workload:
    def __init__(self, name, lib, torch, dev):
        from separableflowthesis_amd import MemorySaver, _lib
        self.name, self.lib, self.torch = name, lib, torch
        B, H, W, Kp, ops = WORKLOADS[name]
        self.B, self.H, self.W, self.Kp, self.ops = B, H, W, Kp, ops
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        self.base_alloc = torch.cuda.memory_allocated()
        f1c, f2c, gr, att = make_inputs(B, H, W, Kp, torch)
        f1, f2 = f1c.to(dev), f2c.to(dev)
        gr = {k: v.to(dev) for k, v in gr.items()}
        E = lambda *s, dt=torch.float32: torch.empty(*s, dtype=dt, device=dev)
        out_u, out_v = E(B, H, W, 2, H), E(B, H, W, 2, W)
        am_u, am_v = E(B, H, W, 1, H, dt=torch.int32), E(B, H, W, 1, W, dt=torch.int32)
        backward = "C" in ops or "F" in ops
        nws = lib.sepcorr_backward_workspace_bytes(B, H, W, H, W, C) if backward else 0
        ws = torch.empty(max(nws, 256), dtype=torch.uint8, device=dev)
        self.workspace_bytes = nws
        dims = (B, H, W, H, W, C)
        stream = torch.cuda.current_stream().cuda_stream
        P = lambda t: t.data_ptr()
        chk = _lib.check

        nfw = lib.sepcorr_forward_workspace_bytes(*dims, max(Kp, 2))
        fws = torch.empty(max(nfw, 256), dtype=torch.uint8, device=dev)
        fwp = P(fws) if nfw else None
        self.forward_workspace_bytes = nfw

        def op_f():
            chk(lib.sepcorr_max_argmax_avg_forward(P(f1), P(f2), P(out_u), P(out_v), P(am_u), P(am_v), *dims, fwp, nfw, stream))

        op_f()
        table = {"f": op_f}
        if Kp:
            # attention weights as the caller produces them: Conv3d on the (max,avg) volumes, softmax over the
            # kept axis, back to (B,H1,W1,K',L) (core/corr.py:437-446)
            with torch.no_grad():
                a_u = MemorySaver.attention_forward(out_v, att[0].weight.to(dev).contiguous(), att[0].bias.to(dev))
                a_v = MemorySaver.attention_forward(out_u, att[1].weight.to(dev).contiguous(), att[1].bias.to(dev))
            cu, cv = E(B, H, W, Kp, H), E(B, H, W, Kp, W)
            table["c"] = lambda: chk(lib.sepcorr_compression_forward(P(f1), P(f2), P(a_u), P(a_v), P(cu), P(cv), *dims, Kp, fwp, nfw, stream))
        if "C" in ops:
            d1, d2 = E(B, H, W, C), E(B, H, W, C)
            da_u, da_v = torch.empty_like(a_u), torch.empty_like(a_v)
            table["C"] = lambda: chk(lib.sepcorr_compression_backward(
                P(f1), P(f2), P(a_u), P(a_v), P(gr["g_cu"]), P(gr["g_cv"]), P(d1), P(d2), P(da_u), P(da_v), *dims, Kp,
                P(ws), nws, stream))
        if "F" in ops:
            d1b, d2b = E(B, H, W, C), E(B, H, W, C)
            table["F"] = lambda: chk(lib.sepcorr_max_argmax_avg_backward(
                P(f1), P(f2), P(am_u), P(am_v), P(gr["g_u"]), P(gr["g_v"]), P(d1b), P(d2b), *dims, P(ws), nws, stream))
        self.seq = [table[o] for o in ops]
        self.fused_step = None
        if "C" in ops and "F" in ops:
            # The same job through the entry points that have no counterpart in the reference's two-operator API:
            # weight gradients alone, then one contraction per feature gradient with dL/dS of both operators added
            # (5 sweeps over the volume instead of 7).
            def fused_step():
                table["f"]()
                table["c"]()
                chk(lib.sepcorr_compression_backward(P(f1), P(f2), P(a_u), P(a_v), P(gr["g_cu"]), P(gr["g_cv"]),
                                                     None, None, P(da_u), P(da_v), *dims, Kp, fwp, nfw, stream))
                chk(lib.sepcorr_fused_backward(P(f1), P(f2), P(am_u), P(am_v), P(gr["g_u"]), P(gr["g_v"]),
                                               P(a_u), P(a_v), P(gr["g_cu"]), P(gr["g_cv"]), P(d1), P(d2),
                                               *dims, Kp, P(ws), nws, stream))
            self.fused_step = fused_step

    def step(self):
        for fn in self.seq:
            fn()

    def time(self, fn, steps, warmup):
        torch = self.torch
        # The clocks of an idle GPU settle over some tens of milliseconds of load (the same build: 2.64 ms per step
        # right after 3 steps, 2.59 after 20 and after 50).  Part of the set-up, like building the inputs: the step
        # runs for about 0.1 s, whatever the number of warm-up steps asked for, so that the timed steps see the
        # clocks a training loop sees.
        t_end = time.perf_counter() + SETTLE_SECONDS
        while time.perf_counter() < t_end:
            fn()
            torch.cuda.synchronize()
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps * 1e3

    def kernel_times(self, fn, profile_steps):
        """Per-kernel durations: HIP events recorded by the library on the stream each kernel is launched on."""
        lib, torch = self.lib, self.torch
        lib.sepcorr_profile_enable(1)
        for _ in range(profile_steps):
            fn()
        torch.cuda.synchronize()
        cap = 8192
        names = ctypes.create_string_buffer(1 << 17)
        tms = (ctypes.c_float * cap)()
        n = lib.sepcorr_profile_collect(names, len(names), tms, cap)
        lib.sepcorr_profile_enable(0)
        per = {}
        for nm, t in zip(names.value.decode().split("\n")[:n], list(tms)[:n]):
            per.setdefault(nm, []).append(t)
        return per

    def report(self, steps, warmup, profile_steps):
        torch = self.torch
        B, H, W, Kp, ops = self.B, self.H, self.W, self.Kp, self.ops
        N = H * W
        ms = self.time(self.step, steps, warmup)
        peak = torch.cuda.max_memory_allocated() - self.base_alloc
        Wf = 2.0 * B * N * N * C
        traffic = measured_traffic(self.name)
        kernels = {}
        for nm, ts in self.kernel_times(self.step, max(1, profile_steps)).items():
            avg = sum(ts) / len(ts)
            ent = {"avg_ms": round(avg, 4), "launches_per_step": round(len(ts) / max(1, profile_steps), 2)}
            if nm in SWEEP_KERNELS:
                ent["tflops"] = round(Wf / (avg * 1e-3) / 1e12, 2)
                ent["frac_of_peak"] = round(ent["tflops"] / PEAK_FP32_MFMA_TFLOPS, 4)
            kernels[nm] = ent
        dom = max((k for k in kernels if k in SWEEP_KERNELS),
                  key=lambda k: kernels[k]["avg_ms"] * kernels[k]["launches_per_step"])
        ach = kernels[dom]["tflops"]
        passes = sum(PASSES[o] for o in ops)
        algorithmic = passes * Wf / (ms * 1e-3) / 1e12
        # The max/avg backward may run as gathers of feature rows instead of its two contractions (the library picks
        # the faster way for the sizes): `tflops` counts the passes that actually ran on the matrix cores; the
        # algorithmic work of the step, 2*B*N1*N2*C per pass of the reference's formulation, over the same time is
        # reported next to it, together with the same step timed with the dense max/avg backward.
        gathered = any(k.endswith("_gather") for k in kernels)
        executed = passes - (PASSES["F"] if gathered else 0)
        value = executed * Wf / (ms * 1e-3) / 1e12
        dense = None
        if gathered:
            prev_mode = self.lib.sepcorr_set_max_avg_backward(1)
            try:
                dms = self.time(self.step, steps, warmup)
            finally:
                self.lib.sepcorr_set_max_avg_backward(prev_mode)
            dense = {"ms_per_step": round(dms, 4), "tflops": round(passes * Wf / (dms * 1e-3) / 1e12, 3),
                     "frac_of_fp32_mfma_peak": round(passes * Wf / (dms * 1e-3) / 1e12 / PEAK_FP32_MFMA_TFLOPS, 4),
                     "what": "the same step with sepcorr_set_max_avg_backward(SEPCORR_MAXAVG_DENSE): every pass a contraction"}
        roofline = {"bound": "mfma", "kernel": dom, "achieved": ach, "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(ach / PEAK_FP32_MFMA_TFLOPS, 4), "traffic": traffic.get(dom),
                    "algorithmic_bytes": algorithmic_bytes(dom, B, N, H, W, Kp),
                    "algorithmic_flop": Wf, "avg_launch_ms": kernels[dom]["avg_ms"]}
        return {
            "workload": f"{self.name}: B={B}, C={C}, {H}x{W}, K'={Kp}, ops={ops}",
            "ms_per_step": round(ms, 4), "tflops": round(value, 3),
            "frac_of_fp32_mfma_peak": round(value / PEAK_FP32_MFMA_TFLOPS, 4),
            "contraction_passes": passes, "gflop_per_step": round(passes * Wf / 1e9, 2),
            "contraction_passes_executed": executed,
            "algorithmic_tflops": round(algorithmic, 3),
            "max_avg_backward": ("gather" if gathered else "dense") if "F" in ops else None,
            "all_dense": dense,
            "note": ("tflops / frac_of_fp32_mfma_peak count the contraction_passes_executed passes that ran on the matrix "
                     "cores; the max/avg backward ran as gathers of feature rows instead of its two contractions; "
                     "algorithmic_tflops counts all contraction_passes of the reference's formulation over the same time; "
                     "all_dense is the same step with every pass a contraction")
                    if gathered else None,
            "peak_hbm_allocated_mib": round(peak / _MIB, 1),
            "backward_workspace_mib": round(self.workspace_bytes / _MIB, 1),
            "forward_workspace_mib": round(self.forward_workspace_bytes / _MIB, 1),
            "volume_4d_never_allocated_mib": round(B * N * N * 4 / _MIB, 1),
            "roofline": roofline, "kernels": kernels,
        }


# ------------------------------------------------------------------------------------------------
# caller level (extras, never `value`)
# ------------------------------------------------------------------------------------------------

SETTLE_SECONDS = 0.1   # untimed load before every timed loop (see Workload.time)


def module_level(name, torch, dev, reps=20, backward=True, warmup=5):
    """The caller's whole separate() over 4 pyramid levels through the drop-in classes: NHWC copies, both operators
    per level, the attention producer and volume assembly, torch autograd; with the peak memory it allocates next to
    what the stored 4D pyramid alone would take (the comparison of scripts/test_model.py:320-382 for this block)."""
    from separableflowthesis_amd import AlternateCorrBlockSepflow
    B, H, W, Kp, _ = WORKLOADS[name]
    g = torch.Generator().manual_seed(1234)
    fmap1 = torch.randn(B, C, H, W, generator=g).to(dev).requires_grad_()
    fmap2 = torch.randn(B, C, H, W, generator=g).to(dev).requires_grad_()
    torch.manual_seed(1234)
    att = tuple(torch.nn.Conv3d(2, Kp, 3, padding=1).to(dev) for _ in range(2)) if Kp else None

    ups = {}   # upstream gradients: dense tensors, as the layers above the block hand them down

    def run(bw):
        with torch.set_grad_enabled(bw):
            blk = AlternateCorrBlockSepflow(fmap1, fmap2, None, 4, 4, support_backward=bw)
            c1, c2 = blk(None, sep=True, attention_weights=att)
            if bw:
                if not ups:
                    ups["g"] = [torch.randn(c.shape, generator=g).to(dev) for c in (c1, c2)]
                # as a training step does before its backward pass (optimizer.zero_grad(), which drops the tensors):
                # the gradients are then stored, not added to those of the previous repeat
                for t in (fmap1, fmap2) + tuple(p for m in (att or ()) for p in m.parameters()):
                    t.grad = None
                torch.autograd.backward([c1, c2], ups["g"])

    out = {}
    for key, bw in (("forward", False), ("forward_backward", True)):
        if bw and not backward:
            continue
        t_end = time.perf_counter() + SETTLE_SECONDS   # (clocks of an idle GPU: see Workload.time)
        while time.perf_counter() < t_end:
            run(bw)
            torch.cuda.synchronize()
        for _ in range(warmup):
            run(bw)
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        t0 = time.perf_counter()
        for _ in range(reps):
            run(bw)
        torch.cuda.synchronize()
        out[key + "_ms"] = round((time.perf_counter() - t0) / reps * 1e3, 3)
        out[key + "_peak_allocated_mib"] = round((torch.cuda.max_memory_allocated() - base) / _MIB, 1)
    n = H * W
    out["returned_volumes_mib"] = round(B * 4 * (2 + Kp) * (H + W) * n * 4 / _MIB, 1)
    out["stored_4d_pyramid_would_take_mib"] = round(B * n * n * 4 * (1 + 1 / 4 + 1 / 16 + 1 / 64) / _MIB, 1)
    out["what"] = f"AlternateCorrBlockSepflow.separate, 4 levels, B={B}, C={C}, {H}x{W}, K'={Kp}, torch autograd around the native ops"
    return out


def lookup_level(B, H, W, torch, dev, reps=20):
    """corr_fn(coords) of the block without the 4D volume: 4 levels, radius 4, a smooth flow field; and CorrBlock1D.
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
    one_d = {}
    for dim in (1, 24):   # one aggregated channel as in the model, and all 24 channels of separate()
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
                              "volumes_mib": round((c1.numel() + c2.numel()) * 4 / _MIB, 1)}
        del c1, c2, u
    pts = B * H * W * 4 * 100                       # (pixel, level, grid point) pairs: one C-long dot product each
    alg = (f1.numel() + sum(t.numel() for t in f2s) + coords.numel() + up.numel()) * 4   # up has the output's size
    return {
        "forward_ms": round(fwd, 4), "backward_ms": round(bwd, 4),
        "forward_window_gb_s": round(pts * C * 4 / fwd / 1e6, 1),
        "forward_algorithmic_mib": round(alg / _MIB, 1),
        "forward_hbm_gb_s": round(alg / fwd / 1e6, 1),
        "volumes_1d": one_d,
        "what": f"sepcorr_lookup_forward / sepcorr_lookup_backward, B={B}, C={C}, {H}x{W}, 4 levels, radius 4; "
                "window = bytes of the fmap2 rows under all windows; algorithmic = f1 + pyramid + coords + out once; "
                "volumes_1d = CorrBlock1D on both separated volumes (sepcorr_lookup1d_forward/backward)",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20,
                    help="untimed steps first: the clocks of an idle GPU take some tens of milliseconds to settle")
    ap.add_argument("--workload", default="cfg4", choices=sorted(WORKLOADS),
                    help="the workload `value` is quoted on (the headline metric is cfg4)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the configs table and the caller-level extras")
    ap.add_argument("--profile-steps", type=int, default=5)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three 256 MiB device copies (known traffic) for scaling rocprofv3 FETCH_SIZE/WRITE_SIZE")
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
    if args.only_lookup:
        print(json.dumps({"workload": args.workload, "lookup": lookup_level(B, H, W, torch, dev)}))
        return
    if args.only_module_level:
        print(json.dumps({"workload": args.workload, "module_level": module_level(args.workload, torch, dev)}))
        return
    if args.calibrate_copy:
        src = torch.empty(64 * 2**20, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    wl = Workload(args.workload, lib, torch, dev)
    head = wl.report(args.steps, args.warmup, args.profile_steps)
    out = {
        "metric": METRIC, "value": head["tflops"], "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "settle_seconds_before_warmup": SETTLE_SECONDS,
        "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": head["workload"] + " " + OPS_TEXT,
                   "contraction_passes": head["contraction_passes"], "gflop_per_step": head["gflop_per_step"],
                   "contraction_passes_executed": head["contraction_passes_executed"],
                   "algorithmic_tflops": head["algorithmic_tflops"], "max_avg_backward": head["max_avg_backward"],
                   "all_dense": head["all_dense"], "note": head["note"],
                   "frac_of_fp32_mfma_peak": head["frac_of_fp32_mfma_peak"],
                   "peak_hbm_allocated_mib": head["peak_hbm_allocated_mib"],
                   "backward_workspace_mib": head["backward_workspace_mib"],
                   "volume_4d_never_allocated_mib": head["volume_4d_never_allocated_mib"]},
        "roofline": head["roofline"],
        "kernels": head["kernels"],
    }
    if wl.fused_step is not None:
        fms = wl.time(wl.fused_step, args.steps, args.warmup)
        Wf = head["roofline"]["algorithmic_flop"]
        out["fused_level"] = {
            "ms_per_step": round(fms, 4), "contraction_passes_executed": 5,
            "tflops_executed": round(5 * Wf / (fms * 1e-3) / 1e12, 2),
            "what": "same inputs and outputs as the headline step (d_f1, d_f2 are the sums of the two operators' "
                    "gradients), via sepcorr_compression_backward(d_f1=d_f2=NULL) + sepcorr_fused_backward"}
        # The headline step with the forward sweeps and d_f1 contracting in three bf16 planes per operand: an option
        # of this library (sepcorr_set_contraction), not the headline arithmetic, which is fp32 MFMA throughout.
        prev_mode = lib.sepcorr_set_contraction(1)
        try:
            pms = wl.time(wl.step, args.steps, args.warmup)
        finally:
            lib.sepcorr_set_contraction(prev_mode)
        out["bf16_planes"] = {"ms_per_step": round(pms, 4),
                              "what": "optional bf16x3 contraction for the forward sweeps and d_f1 (d_f2 stays fp32 MFMA); "
                                      "reported for information, never the headline"}
    del wl
    gc.collect()
    torch.cuda.empty_cache()

    if not args.no_extras:
        # every benchmark configuration, measured in this run (fewer steps than the headline for the small ones is
        # not needed: all of them take milliseconds)
        table = {}
        for name in sorted(WORKLOADS):
            if name == args.workload:
                row = dict(head)
            else:
                w = Workload(name, lib, torch, dev)
                row = w.report(min(args.steps, 20), args.warmup, min(args.profile_steps, 3))
                del w
                gc.collect()
                torch.cuda.empty_cache()
            row["kernels"] = {k: v["avg_ms"] for k, v in row["kernels"].items()}
            table[name] = row
        out["configs"] = table
        out["module_level"] = module_level(args.workload, torch, dev)
        # peak memory of the block that never stores the volume, next to the stored 4D pyramid, per configuration
        mem = {}
        for name in ("cfg3", "cfg4", "cfg5"):
            m = out["module_level"] if name == args.workload else module_level(name, torch, dev, reps=2, backward=name != "cfg5", warmup=2)
            mem[name] = {k: v for k, v in m.items() if k.endswith("_mib")}
            torch.cuda.empty_cache()
        out["memory"] = mem
        out["lookup"] = lookup_level(B, H, W, torch, dev)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, args.workload)
        if "memory" in out:
            # the stored-volume path beside the block, measured on this GPU (a baseline like the CPU timing above)
            for name, ent in stored_volume_path_memory(torch, dev).items():
                out["memory"][name].update(ent)
            out["memory"]["what"] = ("peak of torch's allocator above what is held before the call: the block that never stores the "
                                     "volume (forward_*, forward_backward_*) beside the stored-volume path (stored_4d_path_*: the "
                                     "oracle's CorrBlock4D through torch autograd on this GPU); stored_4d_pyramid_would_take_mib is "
                                     "the size of the 4D pyramid alone")
    print(json.dumps(out))


if __name__ == "__main__":
    main()
