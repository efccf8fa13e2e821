#!/usr/bin/env python3
"""Benchmark of the MoE layer forward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3_mixtral]

A step is one forward of the whole layer (gate -> count/scan/pos -> FFN1+GELU ->
FFN2 -> combine) over one synthetic batch already resident in HBM, issued as a
single C-ABI call.  Prints ONE JSON line: layer tokens/s as ``value``; the
grouped-GEMM TFLOP/s and its fraction of the fp16 dense MFMA peak; a
``roofline`` object for the dominant kernel, timed with HIP events recorded on
the layer's stream inside the timed region; and ``cpu_baseline``, the same
layer through torch on this box's host cores.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP16_TFLOPS = 2500.0          # MI355X dense fp16 MFMA
PEAK_HBM_GBS = 8000.0

# Bytes moved between L2 and the memory fabric per grouped GEMM come from two `rocprofv3 --pmc`
# runs of this script (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch), each scaled by what the
# counter reads for a plain 256 MiB device copy in the same run.  Counters cannot be read from
# inside a normal run, so the figures are parsed from the committed summary
# profiles/grouped_gemm_<workload>_hbm_traffic.txt (its last line, "TRAFFIC ..."), which also
# records a hash of the kernel sources it was measured on: when the sources have changed since,
# the line says so ("traffic_stale": true).  A workload without a summary reports null.
KERNEL_SOURCES = ("ccfuser_amd/csrc/ffn.hip", "ccfuser_amd/csrc/gemm_tile.h", "ccfuser_amd/csrc/plan.h")


def kernel_sources_hash():
    import hashlib
    h = hashlib.sha256()
    for rel in KERNEL_SOURCES:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(workload, stage):
    """(bytes per launch, stale flag, file) from the profile summary, or (None, None, None)."""
    rel = f"profiles/grouped_gemm_{workload}_hbm_traffic.txt"
    path = os.path.join(ROOT, rel)
    if not os.path.exists(path):
        return None, None, None
    rec = None
    for ln in open(path):
        if ln.startswith("TRAFFIC "):
            rec = dict(kv.split("=", 1) for kv in ln.split()[1:])
    if rec is None or f"{stage}_fetch_kib" not in rec:
        return None, None, rel
    nbytes = (float(rec[f"{stage}_fetch_kib"]) * float(rec["fetch_scale"]) +
              float(rec[f"{stage}_write_kib"]) * float(rec["write_scale"])) * 1024.0
    return nbytes, rec.get("sources") != kernel_sources_hash(), rel


def dense_hgemm_ceiling(rows, d, f, steps=30, warmup=15):
    """What the vendor's dense fp16 GEMM (hipBLASLt through torch.matmul) sustains on this box,
    in this process, on the two GEMM shapes of the workload with random operands: rows x d x f
    (FFN1's) and rows x f x d (FFN2's), weights stored [N, K] as the layer stores them.  Reported
    beside the nominal peak: a measured ceiling for a dense, unragged GEMM of the same size."""
    import torch
    g = torch.Generator(device="cuda").manual_seed(7)
    out = {}
    for name, (K, N) in (("ffn1_shape", (d, f)), ("ffn2_shape", (f, d))):
        a = torch.randn(rows, K, device="cuda", generator=g).half()
        w = (torch.randn(N, K, device="cuda", generator=g) * 0.02).half()
        for _ in range(warmup):
            torch.matmul(a, w.t())
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            torch.matmul(a, w.t())
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        tf = 2.0 * rows * K * N / (ms * 1e-3) / 1e12
        out[name] = {"m": rows, "n": N, "k": K, "ms": ms, "tflops": tf, "frac_of_peak": tf / PEAK_FP16_TFLOPS}
        del a, w
    mean = sum(v["tflops"] for v in out.values()) / 2
    out["tflops"] = mean
    out["frac_of_peak"] = mean / PEAK_FP16_TFLOPS
    out["what"] = f"torch.matmul (hipBLASLt) fp16, random operands, {warmup} warm-up + {steps} timed calls per shape"
    return out


def mfma_only_ceiling(lib, seconds=0.15):
    """What the matrix cores sustain with nothing else in the way (ccf_probe_mfma: one workgroup
    per CU, MFMAs on register operands, no memory traffic), with random and with constant
    operands: each launch repeated until `seconds` have passed, the last launches timed."""
    import ctypes as C
    import torch
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    out = torch.empty(cus * 256, dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    res = {}
    for name, const in (("random_operands", 0), ("constant_operands", 1)):
        flop = C.c_double()
        iters = 2000                                              # ~2 ms per launch
        t_end = time.perf_counter() + seconds
        while time.perf_counter() < t_end:                        # lets the clock settle under this load
            lib.ccf_probe_mfma(cus, iters, const, out.data_ptr(), C.byref(flop), stream)
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            lib.ccf_probe_mfma(cus, iters, const, out.data_ptr(), C.byref(flop), stream)
        e1.record()
        torch.cuda.synchronize()
        tf = 10 * flop.value / (e0.elapsed_time(e1) * 1e-3) / 1e12
        res[name] = {"tflops": tf, "frac_of_peak": tf / PEAK_FP16_TFLOPS}
    res["what"] = (f"v_mfma_f32_16x16x32_f16 back to back on register operands, {cus} workgroups of 4 wavefronts, "
                   "no memory traffic")
    return res


class HipEvents:
    """hipEvent_t handles through the HIP runtime (torch's events hide the handle)."""

    def __init__(self):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p,
                                                 ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]

    def create(self):
        ev = ctypes.c_void_p()
        rc = self.hip.hipEventCreate(ctypes.byref(ev))
        if rc != 0:
            raise RuntimeError(f"hipEventCreate failed: {rc}")
        return ev

    def elapsed_ms(self, a, b):
        ms = ctypes.c_float()
        rc = self.hip.hipEventElapsedTime(ctypes.byref(ms), a, b)
        if rc != 0:
            raise RuntimeError(f"hipEventElapsedTime failed: {rc}")
        return float(ms.value)

    def destroy(self, ev):
        self.hip.hipEventDestroy(ev)


def cpu_baseline(wl, max_seconds=30.0):
    """The layer through torch on the host cores, fp32 math on the fp16-rounded
    values (the oracle's torch-only form).  1 warm-up + up to 3 timed runs,
    stopping early once ``max_seconds`` is spent."""
    import torch
    from oracle import moe_oracle as O
    t = wl.tensors
    if "seg_start" in t:
        # the expert-parallel share has no gate: the expert FFN over the inbound segments
        f32 = [t[n].float() for n in ("x", "w1", "b1", "w2", "b2")]
        segs = [t[n] for n in ("seg_start", "seg_len", "seg_expert")]
        run = lambda: O.ffn_segments(f32[0], *segs, *f32[1:])
    else:
        args = [t[n].float() for n in ("x", "wg", "bg", "w1", "b1", "w2", "b2")]
        run = lambda: O.reference_layer_torch(*args, wl.top_k, capacity=wl.capacity)
    threads = torch.get_num_threads()
    with torch.no_grad():
        t0 = time.perf_counter()
        run()
        first = time.perf_counter() - t0
        times = []
        spent = first
        while len(times) < 3 and (not times or spent + times[-1] < max_seconds):
            t0 = time.perf_counter()
            run()
            times.append(time.perf_counter() - t0)
            spent += times[-1]
    med = sorted(times)[len(times) // 2]
    return {"value": wl.tokens / med, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"full {wl.name} batch ({wl.tokens} tokens), fp32 torch on {threads} threads, "
                      f"1 warm-up + median of {len(times)} runs",
            "ms_per_step": med * 1e3}


def bench_backward(a, wl, ops):
    """One training step of the layer: forward in grad mode (gate, FFN1 with the GELU in its
    epilogue and the pre-activation kept, FFN2, combine) and the backward of all of it, K times;
    then the two expert-GEMM backward calls alone, with events around each."""
    import torch
    from ccfuser_amd.mix_moe import MixMOETransformerMLP
    t = wl.tensors
    T, d, f, E, k = wl.tokens, wl.d_model, wl.d_ffn, wl.num_expert, wl.top_k
    K, W = a.steps, a.warmup
    cf = None if wl.capacity < 0 else wl.capacity * E / (T * k)
    mlp = MixMOETransformerMLP("naive", {"num_local_expert": E, "hidden_size": f}, d, 0, 1,
                               total_batch_size=T, top_k=k, capacity_factor=cf,
                               popular_expert_num=0).half().cuda()
    with torch.no_grad():
        mlp.gate.gate.weight.copy_(t["wg"]); mlp.gate.gate.bias.copy_(t["bg"])
        mlp.experts.htoh4.weight.copy_(t["w1"]); mlp.experts.htoh4.bias.copy_(t["b1"])
        mlp.experts.h4toh.weight.copy_(t["w2"]); mlp.experts.h4toh.bias.copy_(t["b2"])
    x = t["x"].cuda().requires_grad_(True)
    gout = torch.randn(T, d, device="cuda", generator=torch.Generator(device="cuda").manual_seed(1)).half()

    def step():
        mlp.zero_grad(set_to_none=True)
        x.grad = None
        mlp(x).backward(gout)

    for _ in range(W):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / K * 1e3

    # the expert-GEMM backward calls alone, preallocated outputs
    with torch.no_grad():
        idx, _ = mlp.gate(x.detach())
        rt = ops.route(idx.reshape(-1), E, k, wl.capacity)
        routed = int(rt["offsets"][-1].item())
        n = T * k
        act = torch.randn(n, f, device="cuda").half()
        gh = torch.randn(n, f, device="cuda").half()
        gy = torch.randn(n, d, device="cuda").half()
        w1, w2 = mlp.experts.htoh4.weight.detach(), mlp.experts.h4toh.weight.detach()
        gw1, gw2 = torch.empty_like(w1), torch.empty_like(w2)
        gb1 = torch.empty(E, f, dtype=torch.float16, device="cuda")
        gb2 = torch.empty(E, d, dtype=torch.float16, device="cuda")
        drop = wl.capacity >= 0                          # without a capacity limit every output row is written: no zero fill
        calls = {"ffn2_backward": lambda: ops.ffn2_backward(gy, act, rt["dst_row"], rt["offsets"], n, w2, gw2, gb2,
                                                            may_drop=drop),
                 "ffn1_backward": lambda: ops.ffn1_backward(gh, x.detach(), rt["src_row"], rt["dst_row"],
                                                            rt["offsets"], n, w1, n, gw1, gb1, may_drop=drop)}
        stage_ms = {}
        for name, fn in calls.items():
            for _ in range(max(2, W)):
                fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(K):
                fn()
            e1.record()
            torch.cuda.synchronize()
            stage_ms[name] = e0.elapsed_time(e1) / K
    gemm_flop = 4.0 * routed * d * f                    # per backward call: input-gradient + weight-gradient GEMM
    dom = max(stage_ms, key=stage_ms.get)
    ach = gemm_flop / (stage_ms[dom] * 1e-3) / 1e12
    step_flop = 12.0 * routed * d * f
    line = {
        "metric": "moe_layer_fwd_bwd_tokens_per_s", "value": T / (ms * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"{wl.name}: {wl.description}; forward + backward", "tokens": T, "top_k": k,
                   "num_expert": E, "d_model": d, "d_ffn": f, "routed_rows": routed,
                   "capacity": wl.capacity, "seed": wl.seed},
        "gemm_tflops": step_flop / (ms * 1e-3) / 1e12,
        "frac_fp16_mfma_peak": step_flop / (ms * 1e-3) / 1e12 / PEAK_FP16_TFLOPS,
        "stages_ms": stage_ms,
        "roofline": {"kernel": f"{dom}: input-gradient and weight-gradient grouped GEMMs with their transposes",
                     "bound": "mfma", "achieved": ach, "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                     "frac": ach / PEAK_FP16_TFLOPS, "traffic": None,
                     "flop_per_launch": gemm_flop, "avg_launch_ms": stage_ms[dom]},
    }
    print(json.dumps(line))


def bench_overlap(a, wl, ops):
    """Does the gate + count/scan/pos of a layer hide under the work in front of it?  The
    reference plans the next MoE layer on a Python thread while attention runs
    (transformer.py:102-145, 376-423); here the planning is a few kernels on a side stream.
    Timed: a dense fp16 GEMM of the layer's token count (standing in for the block in front,
    [T, d] x [d, d]) followed by the staged layer forward, with the assignment issued inline,
    and with it issued on the side stream before the GEMM."""
    import torch
    from ccfuser_amd.mix_moe import MixMOETransformerMLP
    t = wl.tensors
    T, d, f, E, k = wl.tokens, wl.d_model, wl.d_ffn, wl.num_expert, wl.top_k
    K, W = a.steps, a.warmup
    cf = None if wl.capacity < 0 else wl.capacity * E / (T * k)
    mlp = MixMOETransformerMLP("naive", {"num_local_expert": E, "hidden_size": f}, d, 0, 1,
                               total_batch_size=T, top_k=k, capacity_factor=cf, fused=False,
                               popular_expert_num=0).half().cuda()
    with torch.no_grad():
        mlp.gate.gate.weight.copy_(t["wg"]); mlp.gate.gate.bias.copy_(t["bg"])
        mlp.experts.htoh4.weight.copy_(t["w1"]); mlp.experts.htoh4.bias.copy_(t["b1"])
        mlp.experts.h4toh.weight.copy_(t["w2"]); mlp.experts.h4toh.bias.copy_(t["b2"])
    x = t["x"].cuda()
    g = torch.Generator(device="cuda").manual_seed(3)
    pa = torch.randn(T, d, device="cuda", generator=g).half()
    pb = (torch.randn(d, d, device="cuda", generator=g) * 0.02).half()
    pc = torch.empty(T, d, device="cuda", dtype=torch.float16)

    def front():
        torch.matmul(pa, pb, out=pc)

    def inline():
        front()
        return mlp(x)

    def ahead():
        mlp.async_expert_assignment(x)
        front()
        return mlp(x)

    def assign_only():
        mlp.async_expert_assign.capacity = mlp._capacity(T)
        mlp.async_expert_assign.process_data(mlp.gate, x, E, 1)

    out = {}
    with torch.no_grad():
        same = torch.equal(inline(), ahead())
        for name, fn in (("front_gemm", front), ("assignment", assign_only), ("inline", inline), ("ahead", ahead)):
            for _ in range(W):
                fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(K):
                fn()
            torch.cuda.synchronize()
            out[name] = (time.perf_counter() - t0) / K * 1e3
    line = {
        "metric": "moe_layer_with_assignment_ahead_ms", "value": out["ahead"], "unit": "ms",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": out["ahead"], "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"{wl.name}: {wl.description}; a [T,d]x[d,d] GEMM in front of the staged layer "
                               "forward, gate + count/scan/pos inline or on a side stream ahead of that GEMM"},
        "ms": out, "hidden_us": (out["inline"] - out["ahead"]) * 1e3, "outputs_bit_equal": bool(same),
    }
    print(json.dumps(line))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="c3_mixtral")
    ap.add_argument("--no-steady-state", action="store_true",
                    help="with fewer than 45 steps in all: do not run on to time the step after the clock ramp")
    ap.add_argument("--stage-events", choices=("timed", "after"), default="timed",
                    help="record the per-stage HIP events inside the timed steps, or in a second pass of the same steps")
    ap.add_argument("--gemm-variant", type=int, default=None)
    ap.add_argument("--option", action="append", default=[], metavar="NAME=VALUE",
                    help="ccf_set_option before the run (tuning knobs), may repeat")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-dense-ceiling", action="store_true",
                    help="skip the measured ceilings (vendor dense GEMM on the workload's shapes, MFMA-only loop)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain 256 MiB device copies (a known HBM traffic, for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--backward", action="store_true",
                    help="time a training step (forward + backward through the mirrored module) "
                         "instead of the forward; prints its own metric")
    ap.add_argument("--overlap", action="store_true",
                    help="time the staged forward behind a dense GEMM with the gate and routing issued inline "
                         "and ahead on a side stream; prints its own metric")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU's share only: this build has no collectives or sharding "
              "code, so --gpus must be 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from ccfuser_amd import _lib, ops
    from ccfuser_amd.workloads import make_workload

    if not torch.cuda.is_available():
        print("bench.py needs a GPU: the layer has no CPU path", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    lib = _lib.lib()
    if a.gemm_variant is not None:
        ops.set_option("gemm_variant", a.gemm_variant)
    for item in a.option:
        name, _, value = item.partition("=")
        ops.set_option(name, int(value))

    wl = make_workload(a.workload)
    if wl.dtype != torch.float16:
        for k, v in wl.tensors.items():
            if v.is_floating_point():
                wl.tensors[k] = v.half()
    t = wl.tensors
    T, d, f, E, k = wl.tokens, wl.d_model, wl.d_ffn, wl.num_expert, wl.top_k
    ev = HipEvents()
    K, W = a.steps, a.warmup
    stream = torch.cuda.current_stream().cuda_stream

    if a.backward:
        return bench_backward(a, wl, ops)
    if a.overlap:
        return bench_overlap(a, wl, ops)

    segments = a.workload == "c4_ep_share"
    if segments:
        names = ("x", "seg_start", "seg_len", "seg_expert", "w1", "b1", "w2", "b2")
        g = [t[n].cuda() for n in names]
        y = torch.zeros(T, d, dtype=torch.float16, device="cuda")
        n_seg = g[1].numel()
        ws = torch.empty(lib.ccf_segments_workspace_bytes(T, n_seg, E, d, f), dtype=torch.uint8, device="cuda")
        x_, s0, s1, s2, w1_, b1_, w2_, b2_ = [v.data_ptr() for v in g]

        def run():
            _lib.call("ccf_moe_ffn_segments", x_, s0, s1, s2, n_seg, T, d, f, E, w1_, b1_, w2_, b2_,
                      y.data_ptr(), ws.data_ptr(), ws.numel(), stream)
    else:
        names = ("x", "wg", "bg", "w1", "b1", "w2", "b2")
        g = [t[n].cuda() for n in names]
        ws = ops.moe_workspace(T, d, f, E, k, "cuda")
        out = torch.empty(T, d, dtype=torch.float16, device="cuda")
        offsets = torch.empty(E + 1, dtype=torch.int32, device="cuda")
        ptrs = [x.data_ptr() for x in g]

        def run():
            _lib.call("ccf_moe_forward", *ptrs, T, d, f, E, k, wl.capacity, out.data_ptr(), None,
                      None, None, None, offsets.data_ptr(), ws.data_ptr(), ws.numel(), stream)

    events = [[ev.create() for _ in range(6)] for _ in range(K)]
    arrs = [(ctypes.c_void_p * 6)(*row) for row in events]
    for _ in range(W):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(K):
        if a.stage_events == "timed":
            _lib.call("ccf_moe_forward_set_events", arrs[i], 6)
        run()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    if a.stage_events == "after":
        # the same K steps once more, now with an event recorded between the stages
        t1 = time.perf_counter()
        for i in range(K):
            _lib.call("ccf_moe_forward_set_events", arrs[i], 6)
            run()
        torch.cuda.synchronize()
        wall_events = time.perf_counter() - t1
    else:
        wall_events = wall
    _lib.call("ccf_moe_forward_set_events", None, 0)
    # Beside the contract's figure: the same step once the clocks have settled.  The chip ramps its clocks over
    # the first ~25 steps of a load, so a run with few warm-up steps times the ramp; such a run (fewer than 45
    # steps in all) goes on until 45 steps have passed since the start and then times 30 more.  Reported as
    # "steady_state", never as "value".
    steady_ms = None
    if W + K < 45 and not a.no_steady_state:
        for _ in range(45 - W - K):
            run()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        for _ in range(30):
            run()
        torch.cuda.synchronize()
        steady_ms = (time.perf_counter() - t2) / 30 * 1e3
    routed = T if segments else int(offsets[-1].item())
    stage_names = ("gate", "route", "ffn1", "ffn2", "combine")
    stage_ms = {n: sum(ev.elapsed_ms(events[i][s], events[i][s + 1]) for i in range(K)) / K
                for s, n in enumerate(stage_names)}
    for row in events:
        for e in row:
            ev.destroy(e)

    if a.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()

    ms = wall / K * 1e3
    flops = wl.flops(routed)
    tflops = flops / (ms * 1e-3) / 1e12
    line = {
        "metric": "moe_layer_forward_tokens_per_s", "value": T / (ms * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": K, "warmup": W, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": f"{wl.name}: {wl.description}", "tokens": T, "top_k": k,
                   "num_expert": E, "d_model": d, "d_ffn": f, "routed_rows": routed,
                   "capacity": wl.capacity, "seed": wl.seed},
        "gemm_tflops": tflops, "frac_fp16_mfma_peak": tflops / PEAK_FP16_TFLOPS,
    }
    line["stages_ms"] = stage_ms
    line["ms_per_step_with_stage_events"] = wall_events / K * 1e3
    if steady_ms is not None:
        line["steady_state"] = {"ms_per_step": steady_ms, "tokens_per_s": T / (steady_ms * 1e-3),
                                "frac_fp16_mfma_peak": flops / (steady_ms * 1e-3) / 1e12 / PEAK_FP16_TFLOPS,
                                "steps": 30, "after_steps": 45,
                                "what": "the same call, timed after the clock ramp of the first ~25 steps; "
                                        "no stage events; not the contract's figure"}
    dom = "ffn1" if stage_ms["ffn1"] >= stage_ms["ffn2"] else "ffn2"
    ach = (flops / 2) / (stage_ms[dom] * 1e-3) / 1e12
    traffic, stale, traffic_file = measured_traffic(wl.name, dom)
    line["roofline"] = {"kernel": f"grouped GEMM of {dom} (all launches between the stage's two events)",
                        "bound": "mfma", "achieved": ach, "peak": PEAK_FP16_TFLOPS, "unit": "TFLOP/s",
                        "frac": ach / PEAK_FP16_TFLOPS,
                        "traffic": traffic, "traffic_unit": "bytes/launch", "traffic_source": traffic_file,
                        "traffic_stale": stale,
                        "flop_per_launch": flops / 2, "avg_launch_ms": stage_ms[dom]}
    if not segments:
        hbm_bytes = T * d * 2 + E * d * 2 + T * k * 10
        line["gate_gbs"] = hbm_bytes / (stage_ms["gate"] * 1e-3) / 1e9
    if not a.no_dense_ceiling:
        ceil = dense_hgemm_ceiling(routed, d, f)
        line["dense_hgemm_ceiling"] = ceil
        line["roofline"]["frac_of_dense_hgemm_ceiling"] = ach / ceil[f"{dom}_shape"]["tflops"]
        mf = mfma_only_ceiling(_lib.probe_lib())
        line["mfma_only_ceiling"] = mf
        line["roofline"]["frac_of_mfma_only_random_operands"] = ach / mf["random_operands"]["tflops"]
    if not a.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(wl)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
