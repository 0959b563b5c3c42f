"""Headline benchmark: VGG16, fp32, batch 128, one MI355X.

A step is one forwardPropagation + backwardPropagation (SGD fused into the backward kernels) on seeded synthetic
data, with the input resident in HBM. The reference's four policies run literally (BASELINE, VDNN_NONE, VDNN_CONV,
VDNN_ALL), followed by the value-preserving variants; `value` is the literal VDNN_ALL's images/s, every
configuration rides along in `policies`.

Each configuration: warm-up steps, then the timed steps with nothing else going on (this is what ms_per_step and
images_per_s come from), then a short pass of the same steps with the library's per-launch HIP events switched on.
From that pass come the kernel table, the roofline entry (the convolution class with the most device time) and, from
the launches' start and end times, how much of the copies' time ran beside kernels of the compute stream.

The CPU baseline is the C checker under oracle/ on the host cores (convolutions as im2col + blocked SGEMM), one
step at the same batch.

Output: ONE line of strict JSON on stdout, a few KB: the metric, the roofline entry, the CPU baseline and a handful of
scalars. Everything else (every configuration's figures, the kernel table) goes to stderr and into the file that
--details names. The default run has nine configurations; --sweep runs the whole table.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_MFMA_PEAK_TFLOPS = 157.3
BF16_MFMA_PEAK_TFLOPS = 2500.0  # dense; the bfloat16-storage runs multiply on the bfloat16 matrix cores
HBM_PEAK_GBS = 8000.0
HOST_LINK_GBS = 56.6            # what hipMemcpyAsync from / to pinned memory reaches on this machine, each way
FLOP_PER_IMAGE = 92.82e9        # 3 passes over 13 convolutions and 3 FC layers
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "igemm_conv_vgg16_b128_pmc_traffic.txt")
PACKED_FRACTION = {False: 0.60, True: 0.63}   # what a plan takes a packed stream to be of its tensor (measured: 0.57 / 0.60)

# the default run: the reference's four policies as they are, BASELINE with fused rectifiers, BASELINE in the
# perf-optimal algorithm mode (the policies above run the memory-optimal one), the two fastest float
# configurations that hold a third of BASELINE's memory (one with the link unused, one that uses it) and one bfloat16 run
DEFAULT_POLICIES = ",".join([
    "BASELINE", "VDNN_NONE", "VDNN_CONV", "VDNN_ALL", "BASELINE+fused", "BASELINE+perf",
    "VDNN_ALL+refined+fused+zvc+budget3.0", "VDNN_ALL+refined+fused+zvc+inplace+recompute+budget4.1",
    "VDNN_ALL+refined+bf16+fused+zvc+keep+inplace+recompute",
])
# --sweep: every configuration of the results table
SWEEP_POLICIES = ",".join([
    "BASELINE", "VDNN_NONE", "VDNN_CONV", "VDNN_ALL",
    "BASELINE+fused", "VDNN_ALL+refined",
    "VDNN_CONV+refined+ahead+fused+zvc", "VDNN_ALL+refined+ahead+fused+zvc",
    "VDNN_ALL+refined+fused+zvc+keep",
    "VDNN_ALL+refined+fused+zvc+budget3.0", "VDNN_ALL+refined+fused+zvc+budget3.3", "VDNN_ALL+refined+fused+zvc+budget4.0",
    "VDNN_ALL+refined+fused+zvc+inplace+budget3.4", "VDNN_ALL+refined+fused+zvc+inplace+recompute+budget4.0",
    "VDNN_ALL+refined+fused+zvc+inplace+recompute+budget4.1", "VDNN_ALL+refined+fused+zvc+inplace+recompute+budget4.2",
    "BASELINE+bf16+fused", "VDNN_ALL+refined+ahead+bf16+fused+zvc", "VDNN_ALL+refined+bf16+fused+zvc+keep",
    "VDNN_ALL+refined+bf16+fused+zvc+budget5.9", "VDNN_ALL+refined+bf16+fused+zvc+keep+inplace+recompute",
    "VDNN_ALL+refined+bf16+fused+zvc+inplace+recompute+budget5.0", "VDNN_ALL+refined+bf16+fused+zvc+inplace+recompute+budget6.0",
    "BASELINE+perf", "BASELINE+fused+perf", "BASELINE+wino", "VDNN_ALL+perf", "VDNN_ALL+refined+fused+zvc+budget3.0+perf",
    "VDNN_ALL+refined+fused+zvc+inplace+recompute+budget4.0+perf",
])


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def measured_traffic():
    """Bytes per launch (L2 fetch + write-back) of the convolution classes, read from the hardware-counter summary kept
    under profiles/ (two `rocprofv3 --pmc` runs of this script; the file says how the counters were scaled)."""
    out = {}
    try:
        for line in open(TRAFFIC_PROFILE):
            m = re.match(r"^(conv_\S+)\s+launches.*traffic/launch.*=\s*([0-9.]+) MB", line)
            if m:
                out[m.group(1)] = float(m.group(2)) * 1e6
    except OSError:
        pass
    return out


def run_config(Network, be, cnn, policy, algo, batch, steps, warmup, profile_steps, **kw):
    from vdnn_implementation_amd import trace_overlap
    net = Network(cnn, policy, algo, batch, seed=1, **kw)
    try:
        for _ in range(warmup):
            assert net.forwardPropagation() == 0 and net.backwardPropagation() == 0
        net.synchronize()
        net.reset_peak()
        t_bytes0, l_bytes0 = be.zvc_traffic(net.context)
        net.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            assert net.forwardPropagation() == 0 and net.backwardPropagation() == 0
        net.synchronize()
        dt = time.perf_counter() - t0
        st = net.stats()
        loss = net.loss()
        t_bytes1, l_bytes1 = be.zvc_traffic(net.context)
        # the same steps again with every launch bracketed by events (at most 2048 launches are timed)
        be.profile_enable(net.context, True)
        for _ in range(profile_steps):
            assert net.forwardPropagation() == 0 and net.backwardPropagation() == 0
        net.synchronize()
        prof = be.profile_collect(net.context)
        intervals = be.profile_intervals(net.context)
        be.profile_enable(net.context, False)
        plan = None
        if kw.get("hbm_budget_bytes"):
            places = net.placement()
            plan = {"budget_gb": kw["hbm_budget_bytes"] / 1e9, "feasible": net.plan_feasible(), "plan_peak_gb": net.plan_peak_bytes() / 1e9, "offload_lag": net.offload_lag(),
                    "on_device": places.count(1), "packed_on_device": places.count(2), "over_the_link": places.count(3)}
    finally:
        net.close()
    untimed = prof.pop("untimed", {"launches": 0})["launches"]
    res = {"ms_per_step": dt * 1e3 / steps, "images_per_s": batch * steps / dt, "loss": loss,
           "peak_hbm_gb": st["peak_bytes_in_use"] / 1e9, "offload_gb_per_step": st["offload_bytes"] / 1e9,
           "prefetch_gb_per_step": st["prefetch_bytes"] / 1e9, "pinned_gb": st["pinned_bytes"] / 1e9}
    if plan:
        res["plan"] = plan
    # bytes that cross the link each way per step: tensors copied whole, plus the packed streams' bytes
    packed_tensor = (t_bytes1 - t_bytes0) / steps
    packed_link = (l_bytes1 - l_bytes0) / steps
    # (packed tensors that stay on the device are counted by neither offload_bytes nor the link counter, bar what did not fit)
    whole = max(st["offload_bytes"] - (packed_tensor if packed_link > 0.001 * packed_tensor else 0.0), 0.0)
    link = whole + packed_link
    res["link_gb_each_way_per_step"] = link / 1e9
    res["link_ms_each_way"] = link / (HOST_LINK_GBS * 1e9) * 1e3
    if packed_tensor and packed_link > 0.001 * packed_tensor:
        res["zvc_link_bytes_per_tensor_byte"] = packed_link / packed_tensor
    ov = trace_overlap.summarize(trace_overlap.from_profile(intervals))
    timed = sum(v["launches"] for v in prof.values())
    share = timed / max(timed + untimed, 1)
    steps_seen = profile_steps * share
    res["profile_pass"] = {"steps": profile_steps, "launches_timed_share": share,
                           "kernel_busy_ms_per_step": ov["compute_busy"] / max(steps_seen, 1e-9)}
    if ov["copy_busy"] > 0:
        copies = lambda keys: [prof[k] for k in keys if k in prof]
        rate = lambda keys: (sum(c["bytes"] for c in copies(keys)) / max(sum(c["ms"] for c in copies(keys)), 1e-9) / 1e6) if copies(keys) else None
        res["profile_pass"].update({
            "copy_busy_ms_per_step": ov["copy_busy"] / steps_seen, "copy_beside_kernels_ms_per_step": ov["copy_beside_compute"] / steps_seen,
            "overlap_fraction": ov["overlap_fraction"], "both_directions_at_once_ms_per_step": ov["duplex"] / steps_seen,
            "d2h_tensor_gbs": rate(("offload_d2h", "offload_zvc", "offload_zvc_copy")), "h2d_tensor_gbs": rate(("prefetch_h2d", "prefetch_zvc"))})
    # what no schedule can beat: the kernels back to back, or the link busy all step long in both directions at once
    res["step_bound_ms"] = max(res["profile_pass"]["kernel_busy_ms_per_step"], res["link_ms_each_way"])
    return res, prof


def is_bf16(policy_name):
    return "bf16" in policy_name.split("+")[1:]


def is_perf(policy_name):
    mods = policy_name.split("+")[1:]
    return "perf" in mods or "wino" in mods


def perf_kind(policy_name):
    """0: memory-optimal, 1: perf-optimal, 2: perf-optimal with the Winograd variant (each sums in its own order)."""
    mods = policy_name.split("+")[1:]
    return 2 if "wino" in mods else 1 if "perf" in mods else 0


def best_within(results, base, floor_ratio, need_link):
    """The fastest run that holds at least floor_ratio times less device memory than the fp32 BASELINE (and, with
    need_link, moves something over the link)."""
    if not base:
        return None
    ok = {k: v for k, v in results.items() if base["peak_hbm_gb"] / v["peak_hbm_gb"] >= floor_ratio and k.split("+")[0] != "BASELINE"
          and (not need_link or v["link_gb_each_way_per_step"] > 0.5) and v.get("plan", {}).get("feasible", True)}
    if not ok:
        return None
    k = max(ok, key=lambda n: ok[n]["images_per_s"])
    return {"policy": k, "speed_vs_baseline": ok[k]["images_per_s"] / base["images_per_s"],
            "peak_hbm_reduction": base["peak_hbm_gb"] / ok[k]["peak_hbm_gb"], "images_per_s": ok[k]["images_per_s"],
            "peak_hbm_gb": ok[k]["peak_hbm_gb"], "link_gb_each_way_per_step": ok[k]["link_gb_each_way_per_step"]}


def smallest_within(results, base, speed_floor):
    """The run that holds the least device memory among those at least speed_floor times as fast as the fp32 BASELINE."""
    if not base:
        return None
    ok = {k: v for k, v in results.items() if v["images_per_s"] >= speed_floor * base["images_per_s"] and k.split("+")[0] != "BASELINE"}
    if not ok:
        return None
    k = min(ok, key=lambda n: ok[n]["peak_hbm_gb"])
    return {"policy": k, "speed_vs_baseline": ok[k]["images_per_s"] / base["images_per_s"],
            "peak_hbm_reduction": base["peak_hbm_gb"] / ok[k]["peak_hbm_gb"], "images_per_s": ok[k]["images_per_s"],
            "peak_hbm_gb": ok[k]["peak_hbm_gb"], "link_gb_each_way_per_step": ok[k]["link_gb_each_way_per_step"]}


def zvc_standalone(be):
    """The kernels of the compressed offload alone on the device: a rectified tensor of 411 MB (VGG16 conv2_1's input at
    batch 128 in float; twice the elements in bfloat16), half of its elements zero, five times: packed into a staging
    block, moved to pinned host memory by the copy engine, expanded from there. Rates in bytes of the tensor per second;
    the packing kernel reads the tensor and writes the stream (about 0.53 of it)."""
    import ctypes as C
    import numpy as np
    lib, check = be.lib, be.check
    ctx = be.Context(pool_bytes=6 << 30)
    out = {}
    try:
        for es, dtype in ((4, np.uint32), (2, np.uint16)):
            count = 128 * 64 * 112 * 112 * (4 // es)
            rng = np.random.default_rng(1)
            t = rng.integers(1, 60000, size=count, dtype=np.uint32).astype(dtype)
            t[rng.random(count) < 0.5] = 0
            src, dst = ctx.to_device(t, dtype), ctx.alloc(count * es)
            need = lib.vdnn_zvc_buffer_bytes(count, es)
            stage = ctx.alloc(need)
            host = C.c_void_p()
            check(lib.vdnn_host_alloc_pinned(ctx.handle, C.byref(host), need))
            be.profile_enable(ctx.handle, True)
            for _ in range(5):
                check(lib.vdnn_zvc_offload_staged_async(ctx.handle, host, stage.ptr, need // 2 // 16 * 16 + 65536, src.ptr, count, es,
                                                        None, None, None, None, 0))
                ctx.synchronize()
                check(lib.vdnn_zvc_prefetch_async(ctx.handle, dst.ptr, host, count, es, None))
                ctx.synchronize()
            prof = be.profile_collect(ctx.handle)
            be.profile_enable(ctx.handle, False)
            assert np.array_equal(dst.download((count,), dtype), t)
            out["f32" if es == 4 else "bf16"] = {
                "tensor_mb": count * es / 1e6,
                "pack_ms": prof["offload_zvc_pack"]["ms"] / prof["offload_zvc_pack"]["launches"],
                "pack_gbs": prof["offload_zvc_pack"]["bytes"] / prof["offload_zvc_pack"]["ms"] / 1e6,
                "copy_gbs": prof["offload_zvc_copy"]["bytes"] / prof["offload_zvc_copy"]["ms"] / 1e6,
                "expand_gbs": prof["prefetch_zvc"]["bytes"] / prof["prefetch_zvc"]["ms"] / 1e6}
            check(lib.vdnn_host_free_pinned(ctx.handle, host))
            for b in (src, dst, stage):
                b.free()
    finally:
        ctx.close()
    return out


def library_rates(be):
    """Forward convolutions of three VGG16 layers at batch 128, one kernel at a time, HIP events around ten launches after
    twenty untimed ones:
    this library (float memory-optimal, float perf-optimal, bfloat16; NCHW) beside what the image's vendor libraries
    reach on the same box through PyTorch (`conv2d` with the library's own search switched on, NCHW and channels-last;
    `matmul` at the product shape of the deepest layer and at 8192 cubed). The perf-optimal rows are priced as issued:
    three bfloat16 instructions per float product, a third of the bfloat16 peak. Context for the roofline fractions, not
    part of the path: nothing here is called by the library, and PyTorch is imported by this function only."""
    import ctypes as C
    import numpy as np
    lib, check = be.lib, be.check
    layers = [(64, 64, 224), (256, 256, 56), (512, 512, 28)]
    rows = []
    rng = np.random.default_rng(0)
    for name, dtype, algo, es, peak in (("f32_memory_opt", 0, 0, 4, 157.3), ("f32_perf_opt", 0, 1, 4, 2500.0 / 3), ("bf16", 1, 0, 2, 2500.0)):
        ctx = be.Context(pool_bytes=8 << 30)
        h = ctx.handle
        try:
            check(lib.vdnn_ctx_set_activation_dtype(h, dtype))
            ev = [C.c_void_p(), C.c_void_p()]
            for e in ev:
                check(lib.vdnn_event_create(h, C.byref(e), 1))
            for (c, k, hw) in layers:
                g = be.shape(128, c, hw, hw, k, 3, 3, 1, 1, 1, 1)
                x, y, w, b = ctx.alloc(128 * c * hw * hw * es), ctx.alloc(128 * k * hw * hw * es), ctx.alloc(k * c * 9 * 4), ctx.alloc(k * 4)
                xv = rng.standard_normal(128 * c * hw * hw, dtype=np.float32)   # (random like PyTorch's: the clock follows the data)
                if es == 2:
                    xv = (xv.view(np.uint32) >> 16).astype(np.uint16)
                check(lib.vdnn_memcpy_h2d(h, x.ptr, xv.ctypes.data, xv.nbytes))
                wv = rng.standard_normal(k * c * 9, dtype=np.float32) * np.float32(np.sqrt(2.0 / (c * 9)))
                check(lib.vdnn_memcpy_h2d(h, w.ptr, wv.ctypes.data, wv.nbytes))
                bv = rng.standard_normal(k, dtype=np.float32)
                check(lib.vdnn_memcpy_h2d(h, b.ptr, bv.ctypes.data, bv.nbytes))
                nws = int(lib.vdnn_conv_workspace_bytes_dtype(g, algo, 0, dtype))
                ws = ctx.alloc(max(nws, 256))
                run = lambda: check(lib.vdnn_conv_fwd(h, None, g, algo, x.ptr, w.ptr, b.ptr, y.ptr, ws.ptr if nws else None, nws))
                for _ in range(20):   # (the clock takes some milliseconds of load to come up after the upload)
                    run()
                ctx.synchronize()
                check(lib.vdnn_event_record(h, ev[0], None))
                for _ in range(10):
                    run()
                check(lib.vdnn_event_record(h, ev[1], None)); check(lib.vdnn_event_synchronize(h, ev[1]))
                ms = C.c_float(); check(lib.vdnn_event_elapsed_ms(h, ev[0], ev[1], C.byref(ms)))
                tf = 2.0 * 128 * hw * hw * c * k * 9 / (ms.value / 10) / 1e9
                rows.append({"who": "this library, " + name, "what": "conv %d->%d @%d" % (c, k, hw), "ms": ms.value / 10, "tflops": tf, "of_peak": tf / peak})
                for t in (x, y, w, b, ws):
                    t.free()
        finally:
            ctx.close()
    import torch
    import torch.nn.functional as F
    torch.backends.cudnn.benchmark = True
    dev = "cuda:0"

    def timed(fn):
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(10):
            fn()
        e1.record(); torch.cuda.synchronize()
        return e0.elapsed_time(e1) / 10
    for dt, peak in ((torch.float32, 157.3), (torch.bfloat16, 2500.0)):
        tag = "f32" if dt == torch.float32 else "bf16"
        for (c, k, hw) in layers:
            for fmt, fname in ((torch.contiguous_format, "NCHW"), (torch.channels_last, "channels-last")):
                x = torch.randn(128, c, hw, hw, device=dev, dtype=dt).contiguous(memory_format=fmt)
                w = torch.randn(k, c, 3, 3, device=dev, dtype=dt).contiguous(memory_format=fmt)
                ms = timed(lambda: F.conv2d(x, w, padding=1))
                tf = 2.0 * 128 * hw * hw * c * k * 9 / ms / 1e9
                rows.append({"who": "vendor conv2d, %s %s" % (tag, fname), "what": "conv %d->%d @%d" % (c, k, hw), "ms": ms, "tflops": tf, "of_peak": tf / peak})
                del x, w
        for (m, n, k) in ((512, 100352, 4608), (8192, 8192, 8192)):
            a, b = torch.randn(m, k, device=dev, dtype=dt), torch.randn(k, n, device=dev, dtype=dt)
            ms = timed(lambda: torch.matmul(a, b))
            tf = 2.0 * m * n * k / ms / 1e9
            rows.append({"who": "vendor matmul, %s" % tag, "what": "%d x %d x %d" % (m, n, k), "ms": ms, "tflops": tf, "of_peak": tf / peak})
            del a, b
    return rows


def cpu_baseline(batch, threads):
    """The checker's training step (forward, backward, SGD) on the host cores: VGG16, float."""
    import oracle
    oracle.set_threads(threads)
    oracle.set_blocked_gemm(True)   # convolutions as im2col + cache-blocked SGEMM; the parity tests use the direct loops
    net = oracle.Net(cnn=4, batch=batch)
    net.init_seeded(1)
    t0 = time.perf_counter()
    net.forward()
    net.backward()
    dt = time.perf_counter() - t0
    net.close()
    return {"value": batch / dt, "unit": "images/s", "cores": threads, "kind": "port", "host_cpus_seen": os.cpu_count(),
            "sample": "one VGG16 fp32 step (forward+backward+SGD) at batch %d%s, %.1f s; %s" % (
                batch, "" if batch == 128 else " (the headline's batch is 128)", dt, oracle.build_description())}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--profile-steps", type=int, default=4, help="steps of the pass that times every launch")
    ap.add_argument("--batch", type=int, default=128)
    ap.add_argument("--cnn", default="VGG16", choices=["VGG16", "ALEXNET", "ALEXNET_LRN", "OVERFEAT"], help="the network (the metric is VGG16's)")
    ap.add_argument("--algo", default="VDNN_MEMORY_OPT_ALGO")
    ap.add_argument("--policies", default=None, help="comma-separated configurations (default: eight; see --sweep)")
    ap.add_argument("--sweep", action="store_true", help="run every configuration of the results table (twenty-three)")
    ap.add_argument("--details", default=os.path.join(ROOT, "gpurun_out", "bench_details.json"), help="file that gets every configuration's figures and the kernel table")
    ap.add_argument("--cap-gb", type=float, default=0.0, help="artificial limit on pool bytes in use (0 = none)")
    ap.add_argument("--bf16", action="store_true", help="bfloat16 activation storage in every configuration")
    ap.add_argument("--offload-lag", type=int, default=0, help="layers enqueued before an offloaded block is recycled (0 = reference schedule)")
    ap.add_argument("--prefetch-depth", type=int, default=1, help="offloaded tensors fetched ahead in backward (1 = reference schedule)")
    ap.add_argument("--keep-tail-gb", type=float, default=0.0, help="the deepest offloaded tensors stay on the device, up to this many GB")
    ap.add_argument("--cpu-batch", type=int, default=0, help="batch of the CPU baseline's step (0: 128, the headline's batch; about 15-30 s on 16 threads)")
    ap.add_argument("--cpu-threads", type=int, default=0, help="threads of the CPU baseline (0: the box's CPU share, at most 16)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--zvc-standalone", action="store_true", help="also time the kernels of the compressed offload alone on the device")
    ap.add_argument("--library-rates", action="store_true", help="also time single forward convolutions beside the vendor libraries' (through PyTorch); into --details")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus)
        sys.exit(2)

    import vdnn_implementation_amd.backend as be
    from vdnn_implementation_amd import enums
    from vdnn_implementation_amd.network import Network, parse

    # the headline is VGG16; the other built-in tables are there for profiles of the kernels VGG16 does not have (LRN,
    # overlapping pooling, strided and large-window convolutions)
    cnn = {"VGG16": enums.VGG16_128, "ALEXNET": enums.ALEXNET, "ALEXNET_LRN": enums.ALEXNET_LRN, "OVERFEAT": enums.OVERFEAT}[args.cnn]
    # the fp32 BASELINE's peak, from a replay of its allocation schedule: what the "+budgetX" rows divide by X
    with Network(cnn, enums.BASELINE, 0, args.batch, plan_only=True) as replay:
        assert replay.forwardPropagation() == 0 and replay.backwardPropagation() == 0
        baseline_peak = replay.stats()["peak_bytes_in_use"]

    results, profiles = {}, {}
    policies = args.policies or (SWEEP_POLICIES if args.sweep else DEFAULT_POLICIES)
    for name in policies.split(","):
        # suffixes (none changes a computed value): "+refined" lifetime refinements; "+slack" blocks recycled six layers
        # after their offload and two tensors fetched ahead; "+ahead" the same lag, backward fetches ahead wherever the
        # peak cannot rise; "+fused" ReLU layers run inside the neighbouring layers' kernels; "+zvc" offloaded rectified
        # tensors are packed (no zero elements); "+keep" the packed tensors stay in device memory; "+tail" the deepest
        # 0.75 G elements of the offload set stay on the device; "+budgetX" the policy meets a budget of the fp32
        # BASELINE's peak / X by choosing a place for every tensor; "+bf16" bfloat16 activation storage; "+inplace" input
        # gradients written over the inputs nothing reads again; "+recompute" the first layer's output computed again in
        # backward instead of kept; "+lagN" blocks recycled N layers after their offload
        word, *mods = name.split("+")
        budget = [float(m[6:]) for m in mods if m.startswith("budget")]
        lag_given = [int(m[3:]) for m in mods if m.startswith("lag")]
        link_first = [float(m[4:]) for m in mods if m.startswith("link")]   # "+linkX": X GB each way go over the link before anything is packed on the device
        mods = [m for m in mods if not m.startswith("budget") and not m.startswith("lag") and not m.startswith("link")]
        assert set(mods) <= {"refined", "slack", "bf16", "fused", "zvc", "tail", "ahead", "keep", "inplace", "recompute", "perf", "wino"}, name
        # "+perf": VDNN_PERF_OPT_ALGO, the workspace-using kernel variants (3x3 layers on the bfloat16 matrix cores with every
        # float operand as two bfloat16 parts): other sums than the memory-optimal kernels', so its loss is compared within
        # the mode only. "+wino": the same mode with its Winograd variant where that applies (vdnn_conv_perf_variant).
        _, policy, algo = parse("VGG16_128", word, "VDNN_PERF_OPT_ALGO" if ("perf" in mods or "wino" in mods) else args.algo)
        be.lib.vdnn_conv_perf_variant(1 if "wino" in mods else 0)
        bf16 = args.bf16 or "bf16" in mods
        # (what a plan sends over the link gets the slack that hides it: the plan chooses the offload lag itself - the
        # longest of those that fit with the fewest bytes on the link - and backward fetches ahead wherever the peak allows)
        ahead = "ahead" in mods or bool(budget)
        lag, depth = (6, 2) if "slack" in mods else (-1, 1) if budget else (6, 1) if ahead else (args.offload_lag, args.prefetch_depth)
        if lag_given:
            lag = lag_given[0]
        kw = dict(refined="refined" in mods, in_place="inplace" in mods, recompute_first="recompute" in mods, cap_bytes=int(args.cap_gb * 1e9), bf16=bf16, offload_lag=lag, prefetch_depth=depth,
                  fuse="fused" in mods, compress="zvc" in mods, prefetch_within_peak=ahead, keep_packed="keep" in mods,
                  keep_tail_bytes=int(0.75e9) * (2 if bf16 else 4) if "tail" in mods else int(args.keep_tail_gb * 1e9))
        if budget:
            kw.update(hbm_budget_bytes=int(baseline_peak / budget[0]), plan_packed_fraction=PACKED_FRACTION[bf16])
            if link_first:
                kw.update(plan_link_bytes=int(link_first[0] * 1e9))
        log("[bench] %s %s batch %d: %d warm-up + %d timed + %d profiled steps" % (name, args.algo, args.batch, args.warmup, args.steps, args.profile_steps))
        results[name], profiles[name] = run_config(Network, be, cnn, policy, algo, args.batch, args.steps, args.warmup, args.profile_steps, **kw)
        r = results[name]
        log("[bench]   %.1f ms/step, %.1f img/s, peak %.2f GB, link %.2f GB each way (%.1f ms), overlap %s, loss %.6f%s" % (
            r["ms_per_step"], r["images_per_s"], r["peak_hbm_gb"], r["link_gb_each_way_per_step"], r["link_ms_each_way"],
            "%.2f" % r["profile_pass"]["overlap_fraction"] if r["profile_pass"].get("overlap_fraction") is not None else "-", r["loss"],
            (" plan %s" % json.dumps(r["plan"])) if "plan" in r else ""))

    head = "VDNN_ALL" if "VDNN_ALL" in results else list(results)[0]
    base = results.get("BASELINE")
    # dominant kernel: the convolution class with the most device time over the profiled passes of the runs of the
    # headline's element type
    prof = {}
    headline_bf16 = args.bf16 or all(is_bf16(n) for n in profiles)
    for pname, p in profiles.items():
        if (args.bf16 or is_bf16(pname)) != headline_bf16 or is_perf(pname) != is_perf(head):
            continue   # (the kernel table and the roofline entry are those of the headline's element type and algorithm mode)
        for k, v in p.items():
            acc = prof.setdefault(k, {"launches": 0, "ms": 0.0, "flops": 0.0, "bytes": 0.0})
            for field in acc:
                acc[field] += v[field]
    conv = {k: v for k, v in prof.items() if k.startswith("conv_") and v["flops"] > 0}
    prof = {k: v for k, v in prof.items() if v["ms"] > 0}
    peak = BF16_MFMA_PEAK_TFLOPS if headline_bf16 else FP32_MFMA_PEAK_TFLOPS
    roofline, conv_all_tf = None, None   # (a run with --profile-steps 0, for an outside profiler, times no launch)
    if conv:
        dom = max(conv, key=lambda k: conv[k]["ms"])
        d = conv[dom]
        achieved = d["flops"] / (d["ms"] * 1e-3) / 1e12
        peak = BF16_MFMA_PEAK_TFLOPS if "bf16" in dom else FP32_MFMA_PEAK_TFLOPS
        if "split" in dom:
            # float operands as two bfloat16 parts: three bfloat16 matrix instructions per product, priced as issued
            achieved, peak = 3.0 * achieved, BF16_MFMA_PEAK_TFLOPS
        conv_all_tf = sum((3.0 if "split" in k and "split" in dom else 1.0) * v["flops"] for k, v in conv.items()) / (sum(v["ms"] for v in conv.values()) * 1e-3) / 1e12
        traffic = measured_traffic().get(dom) if args.cnn == "VGG16" and args.batch == 128 and args.algo == "VDNN_MEMORY_OPT_ALGO" and not headline_bf16 else None
        roofline = {"bound": "mfma", "kernel": dom, "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
                    "frac": achieved / peak, "traffic": traffic,
                    "traffic_unit": "bytes/launch, L2 fetch + write-back, profiles/%s" % os.path.basename(TRAFFIC_PROFILE),
                    "algorithmic_flop_per_launch": (3.0 if "split" in dom else 1.0) * d["flops"] / d["launches"],
                    "avg_launch_ms": d["ms"] / d["launches"], "launches": d["launches"]}
    kernels = {k: {"launches": v["launches"], "avg_ms": v["ms"] / max(v["launches"], 1),
                   "tflops": (v["flops"] / (v["ms"] * 1e-3) / 1e12) if v["flops"] else None,
                   "gbs": (v["bytes"] / (v["ms"] * 1e-3) / 1e9) if v["bytes"] else None}
               for k, v in sorted(prof.items(), key=lambda kv: -kv[1]["ms"])}
    fp32 = {k: v for k, v in results.items() if not (args.bf16 or is_bf16(k))}
    same_sums = {k: v for k, v in fp32.items() if perf_kind(k) == perf_kind(head)}   # the headline's algorithm mode: its losses, bit for bit
    ratio = (results[head]["images_per_s"] / base["images_per_s"]) if base and head != "BASELINE" else None

    def brief(b):
        return None if b is None else {"policy": b["policy"], "speed_vs_baseline": round(b["speed_vs_baseline"], 4),
                                       "peak_hbm_reduction": round(b["peak_hbm_reduction"], 3), "peak_hbm_gb": round(b["peak_hbm_gb"], 3),
                                       "link_gb_each_way": round(b["link_gb_each_way_per_step"], 3)}

    # the stdout line: the contract's keys, the roofline entry, the CPU baseline and six figures more
    out = {
        "metric": "VGG16-128 train img/s (VDNN_ALL vs BASELINE); peak HBM GB; conv MFMA util" if args.cnn == "VGG16" else "%s train img/s (not the metric's network)" % args.cnn,
        "value": results[head]["images_per_s"], "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": results[head]["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        # no published figure exists for this metric; the metric itself is a ratio, so this is the literal VDNN_ALL's
        # images/s over BASELINE's, both measured in this run
        "vs_baseline": ratio,
        "dtype": "bf16" if headline_bf16 else "f32", "data": "synthetic",
        "config": {"workload": "%s %s batch %d, one SGD step (fwd+bwd), policy %s, %s" % (args.cnn, "bf16-storage" if headline_bf16 else "fp32", args.batch, head, "VDNN_PERF_OPT_ALGO" if is_perf(head) else args.algo),
                   "batch": args.batch, "policy": head, "algo": args.algo, "configurations_run": len(results)},
        "roofline": roofline,
        "baseline_images_per_s": base["images_per_s"] if base else None,
        "peak_hbm_gb": results[head]["peak_hbm_gb"],
        "peak_hbm_reduction_vs_baseline": (base["peak_hbm_gb"] / results[head]["peak_hbm_gb"]) if base else None,
        # within an element type and an algorithm mode every configuration runs the same kernels on the same values
        "losses_bit_identical": all(len({results[k]["loss"] for k in results if is_bf16(k) == b and perf_kind(k) == p}) <= 1 for b in (False, True) for p in (0, 1, 2)),
        "perf_opt_speed_vs_memory_opt": (results["BASELINE+perf"]["images_per_s"] / base["images_per_s"]) if base and "BASELINE+perf" in results else None,
        "conv_mfma_util": conv_all_tf / peak if conv_all_tf else None,
        # float only, same losses as the literal run bit for bit: the fastest VDNN configuration at >= 3x less memory than
        # BASELINE, and the fastest of those that move at least 0.5 GB over the link each way
        "best_fp32_at_3x": brief(best_within(same_sums, base, 3.0, False)),
        "best_fp32_at_3x_over_the_link": brief(best_within(same_sums, base, 3.0, True)),
    }
    details = {
        "policies": results, "kernels": kernels,
        "least_memory_fp32_at_85pct": smallest_within(fp32, base, 0.85),
        "best_any_dtype_at_3x": best_within(results, base, 3.0, False),
        "best_fp32_any_mode_at_3x": best_within(fp32, base, 3.0, False),   # (the perf-optimal rows sum in another order)
        "baseline_peak_gb_replayed": baseline_peak / 1e9,
        "step_mfma_frac": args.batch * FLOP_PER_IMAGE / (results[head]["ms_per_step"] * 1e-3) / 1e12 / peak if args.cnn == "VGG16" else None,
    }
    if args.zvc_standalone:
        log("[bench] compressed offload alone on the device")
        details["zvc_standalone"] = zvc_standalone(be)
        log("[bench]   %s" % json.dumps(details["zvc_standalone"]))
    if args.library_rates:
        log("[bench] single forward convolutions beside the vendor libraries'")
        details["library_rates"] = library_rates(be)
        for r in details["library_rates"]:
            log("[bench]   %-36s %-26s %8.3f ms %7.0f TFLOP/s  %.2f of peak" % (r["who"], r["what"], r["ms"], r["tflops"], r["of_peak"]))
    if not args.no_cpu_baseline:
        threads = args.cpu_threads or min(16, os.cpu_count() or 1)
        cpu_batch = args.cpu_batch or 128
        log("[bench] CPU baseline: checker, VGG16 batch %d on %d threads" % (cpu_batch, threads))
        out["cpu_baseline"] = cpu_baseline(cpu_batch, threads)
    details["headline"] = out
    log("[bench] details: %s" % json.dumps(details))
    try:
        os.makedirs(os.path.dirname(os.path.abspath(args.details)), exist_ok=True)
        with open(args.details, "w") as f:
            json.dump(details, f, indent=1)
        log("[bench] details written to %s" % args.details)
    except OSError as e:
        log("[bench] details not written (%s)" % e)
    line = json.dumps(out, allow_nan=False)
    assert len(line) < 4096 and "\n" not in line, len(line)
    print(line, flush=True)


if __name__ == "__main__":
    main()
