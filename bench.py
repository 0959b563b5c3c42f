"""Headline benchmark: VGG16, fp32, batch 128, one MI355X.

A step is one forwardPropagation + backwardPropagation (SGD fused into the backward kernels) on
seeded synthetic data. BASELINE, VDNN_NONE, VDNN_CONV and VDNN_ALL run back to back; `value` is the
VDNN_ALL images/s, the other policies and the ratio to BASELINE ride along in `policies`.
The roofline entry is the convolution kernel class with the largest share of device time, timed with
HIP events around every launch on the compute stream during the timed steps. The CPU baseline is the
C checker under oracle/ (a port of the same layer math) on the host cores, at a reduced batch.

One JSON line on stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_MFMA_PEAK_TFLOPS = 157.3
BF16_MFMA_PEAK_TFLOPS = 2500.0  # dense; the bfloat16-storage runs multiply on the bfloat16 matrix cores
HBM_PEAK_GBS = 8000.0
FLOP_PER_IMAGE = 92.82e9  # 3 passes over 13 convolutions and 3 FC layers

# Memory traffic per launch (bytes fetched into L2 plus bytes written back, averaged over a class's
# launches in one step) of the three large convolution classes at the default workload (batch 128,
# memory-optimal mode). Hardware counters cannot be read from inside this script: the figures come
# from two `rocprofv3 --pmc` runs of this script (FETCH_SIZE, then WRITE_SIZE), whose summary is
# kept under profiles/. FETCH_SIZE is scaled by 2.0 and WRITE_SIZE by 1.0: what the same counters
# read for the ReLU kernels of the same run, which move a known number of bytes.
MEASURED_TRAFFIC_BYTES = {
    "conv_fwd_128x128": 984.8e6,
    "conv_bwd_data_128x128": 940.3e6,
    "conv_bwd_filter_128x128": 1724.8e6,
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def run_policy(Network, be, cnn, policy, algo, batch, steps, warmup, seed, refined=False, cap_bytes=0, bf16=False, offload_lag=0, prefetch_depth=1,
               fuse=False, compress=False, keep_tail_bytes=0, ahead=False, keep_packed=False):
    net = Network(cnn, policy, algo, batch, seed=seed, refined=refined, cap_bytes=cap_bytes, bf16=bf16,
                  offload_lag=offload_lag, prefetch_depth=prefetch_depth, fuse=fuse, compress=compress, keep_tail_bytes=keep_tail_bytes, prefetch_within_peak=ahead, keep_packed=keep_packed)
    try:
        for _ in range(warmup):
            assert net.forwardPropagation() == 0 and net.backwardPropagation() == 0
        net.synchronize()
        net.reset_peak()
        be.profile_enable(net.context, True)
        net.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            assert net.forwardPropagation() == 0 and net.backwardPropagation() == 0
        net.synchronize()
        dt = time.perf_counter() - t0
        prof = be.profile_collect(net.context)
        be.profile_enable(net.context, False)
        # the library times the first 2048 launches after profile_enable: the share of the run they stand for
        untimed = prof.pop("untimed", {"launches": 0})["launches"]
        timed = sum(v["launches"] for v in prof.values())
        timed_share = timed / max(timed + untimed, 1)
        st = net.stats()
        loss = net.loss()
        tensor_bytes, link_bytes = be.zvc_traffic(net.context)
    finally:
        net.close()
    res = {"ms_per_step": dt * 1e3 / steps, "images_per_s": batch * steps / dt, "loss": loss,
           "peak_hbm_gb": st["peak_bytes_in_use"] / 1e9, "offload_gb_per_step": st["offload_bytes"] / 1e9,
           "prefetch_gb_per_step": st["prefetch_bytes"] / 1e9, "pinned_gb": st["pinned_bytes"] / 1e9,
           "launches_timed_share": timed_share}
    # host link: busy time and rate of the copies, and how much of the copy time ran under compute
    # (the *_zvc entries are the compacting copies: their bytes are the tensors', not what crossed the link)
    link = ("offload_d2h", "prefetch_h2d", "offload_zvc", "offload_zvc_copy", "prefetch_zvc")   # (not prefetch_zvc_device)
    copies = [prof[k] for k in link if k in prof]
    if tensor_bytes:
        res["zvc_link_bytes_per_tensor_byte"] = link_bytes / tensor_bytes
    if copies:
        copy_ms = sum(c["ms"] for c in copies)
        kernel_ms = sum(v["ms"] for k, v in prof.items() if k not in link)
        rate = lambda keys: (sum(prof[k]["bytes"] for k in keys if k in prof) /
                             max(sum(prof[k]["ms"] for k in keys if k in prof), 1e-9) * 1e3 / 1e9)
        res["d2h_gbs"] = rate(("offload_d2h", "offload_zvc", "offload_zvc_copy"))
        res["h2d_gbs"] = rate(("prefetch_h2d", "prefetch_zvc"))
        copy_ms, kernel_ms = copy_ms / timed_share, kernel_ms / timed_share   # scaled to the whole run
        res["copy_busy_ms_per_step"] = copy_ms / steps
        res["kernel_busy_ms_per_step"] = kernel_ms / steps
        # step = kernels + copies - overlap + idle  =>  overlap >= kernels + copies - step
        res["overlap_fraction_lower_bound"] = max(0.0, min(1.0, (kernel_ms + copy_ms - dt * 1e3) / copy_ms))
    return res, prof


def is_bf16(policy_name):
    return "bf16" in policy_name.split("+")[1:]


def best_offloading(results, base):
    """The offloading run that is fastest among those holding at least 3x less device memory than the fp32 BASELINE."""
    if not base:
        return None
    ok = {k: v for k, v in results.items() if v["offload_gb_per_step"] > 0 and base["peak_hbm_gb"] / v["peak_hbm_gb"] >= 3.0}
    if not ok:
        return None
    k = max(ok, key=lambda n: ok[n]["images_per_s"])
    return {"policy": k, "speed_vs_baseline": ok[k]["images_per_s"] / base["images_per_s"],
            "peak_hbm_reduction": base["peak_hbm_gb"] / ok[k]["peak_hbm_gb"], "images_per_s": ok[k]["images_per_s"],
            "peak_hbm_gb": ok[k]["peak_hbm_gb"]}


def zvc_standalone(be):
    """The compacting kernels alone on the device: a rectified fp32 tensor of conv2_1's input size (half zeros) is packed
    into a staging block, moved by the copy engine, and expanded again from pinned host memory. Rates in bytes of the
    tensor per second; the packing kernel reads the tensor and writes the stream (about 0.53 of it)."""
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
                check(lib.vdnn_zvc_offload_staged_async(ctx.handle, host, stage.ptr, need // 2 // 16 * 16 + 65536, src.ptr, count, es, None, None, None, None, 0))
                ctx.synchronize()
                check(lib.vdnn_zvc_prefetch_async(ctx.handle, dst.ptr, host, count, es, None))
                ctx.synchronize()
            prof = be.profile_collect(ctx.handle)
            be.profile_enable(ctx.handle, False)
            assert np.array_equal(dst.download((count,), dtype), t)
            tensor_bytes, link_bytes = be.zvc_traffic(ctx.handle)
            out["f32" if es == 4 else "bf16"] = {
                "tensor_mb": count * es / 1e6,
                "pack_gbs": prof["offload_zvc_pack"]["bytes"] / prof["offload_zvc_pack"]["ms"] / 1e6,
                "pack_ms": prof["offload_zvc_pack"]["ms"] / prof["offload_zvc_pack"]["launches"],
                "copy_gbs": prof["offload_zvc_copy"]["bytes"] / prof["offload_zvc_copy"]["ms"] / 1e6,
                "expand_gbs": prof["prefetch_zvc"]["bytes"] / prof["prefetch_zvc"]["ms"] / 1e6}
            check(lib.vdnn_host_free_pinned(ctx.handle, host))
            for b in (src, dst, stage):
                b.free()
    finally:
        ctx.close()
    return out


def cpu_baseline(batch):
    """The checker's training step on the host cores, VGG16 at a reduced batch."""
    import oracle
    threads = min(16, os.cpu_count() or 1)
    oracle.set_threads(threads)
    net = oracle.Net(cnn=4, batch=batch)
    net.init_seeded(1)
    t0 = time.perf_counter()
    net.forward()
    net.backward()
    dt = time.perf_counter() - t0
    net.close()
    return {"value": batch / dt, "unit": "images/s", "cores": threads, "kind": "port",
            "sample": "one VGG16 fp32 step (forward+backward+SGD) at batch %d instead of 128, %.1f s" % (batch, dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--batch", type=int, default=128)
    ap.add_argument("--algo", default="VDNN_MEMORY_OPT_ALGO")
    ap.add_argument("--policies", default="BASELINE,VDNN_NONE,VDNN_CONV,VDNN_ALL,VDNN_CONV+refined,VDNN_ALL+refined,VDNN_CONV+refined+slack,"
                    "BASELINE+fused,VDNN_CONV+refined+slack+fused,VDNN_CONV+refined+slack+zvc,VDNN_CONV+refined+ahead+fused+zvc,"
                    "VDNN_CONV+refined+ahead+fused+zvc+tail,VDNN_CONV+refined+slack+fused+zvc+tail,VDNN_ALL+refined+slack+fused+zvc,"
                    "VDNN_ALL+refined+fused+zvc+keep,VDNN_CONV+refined+fused+zvc+keep,"
                    "BASELINE+bf16,VDNN_ALL+bf16,VDNN_CONV+refined+slack+bf16,VDNN_ALL+refined+slack+bf16,"
                    "BASELINE+bf16+fused,VDNN_CONV+refined+slack+bf16+fused,VDNN_CONV+refined+ahead+bf16+fused+zvc+tail,"
                    "VDNN_ALL+refined+slack+bf16+fused+zvc,VDNN_ALL+refined+bf16+fused+zvc+keep,VDNN_CONV+refined+bf16+fused+zvc+keep")
    ap.add_argument("--cap-gb", type=float, default=0.0, help="artificial limit on pool bytes in use (0 = none)")
    ap.add_argument("--bf16", action="store_true", help="bfloat16 activation storage (products on the bfloat16 matrix cores, float accumulation and parameters)")
    ap.add_argument("--offload-lag", type=int, default=0, help="layers enqueued before an offloaded block is recycled (0 = reference schedule)")
    ap.add_argument("--prefetch-depth", type=int, default=1, help="offloaded tensors fetched ahead in backward (1 = reference schedule)")
    ap.add_argument("--keep-tail-gb", type=float, default=0.0, help="the deepest offloaded tensors stay on the device, up to this many GB")
    ap.add_argument("--cpu-batch", type=int, default=24)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--zvc-standalone", action="store_true", help="also time the compacting kernels alone on the device")
    args = ap.parse_args()
    if args.gpus != 1:
        log("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % args.gpus)
        sys.exit(2)

    import vdnn_implementation_amd.backend as be
    from vdnn_implementation_amd import enums
    from vdnn_implementation_amd.network import Network, parse

    cnn = enums.VGG16_128
    results, profiles = {}, {}
    for name in args.policies.split(","):
        # suffixes: "+refined" = the value-preserving lifetime refinements; "+slack" = blocks recycled six layers
        # after their offload and two tensors fetched ahead; "+bf16" = bfloat16 activation storage; "+fused" = ReLU
        # layers run inside the neighbouring layers' kernels; "+zvc" = offloaded rectified tensors cross the link
        # without their zero elements (lossless)
        word, *mods = name.split("+")
        # "+tail" = the deepest offloaded tensors, 0.75 G elements of them, stay on the device
        # "+ahead" = backward fetches ahead wherever the peak cannot rise, blocks recycled six layers after their offload
        # "+keep" = with zvc: the packed tensors stay in device memory instead of crossing the link
        assert set(mods) <= {"refined", "slack", "bf16", "fused", "zvc", "tail", "ahead", "keep"}, name
        _, policy, algo = parse("VGG16_128", word, args.algo)
        lag, depth = (6, 2) if "slack" in mods else (6, 1) if "ahead" in mods else (args.offload_lag, args.prefetch_depth)
        log("[bench] %s %s batch %d: %d warm-up + %d timed steps" % (name, args.algo, args.batch, args.warmup, args.steps))
        results[name], profiles[name] = run_policy(Network, be, cnn, policy, algo, args.batch, args.steps, args.warmup, seed=1,
                                                   refined=("refined" in mods), cap_bytes=int(args.cap_gb * 1e9),
                                                   bf16=(args.bf16 or "bf16" in mods), offload_lag=lag, prefetch_depth=depth,
                                                   fuse=("fused" in mods), compress=("zvc" in mods), ahead=("ahead" in mods), keep_packed=("keep" in mods), keep_tail_bytes=(int(0.75e9) * (2 if (args.bf16 or "bf16" in mods) else 4) if "tail" in mods
                                                                    else int(args.keep_tail_gb * 1e9)))
        log("[bench]   %.1f ms/step, %.1f img/s, peak %.2f GB, loss %.6f" % (
            results[name]["ms_per_step"], results[name]["images_per_s"], results[name]["peak_hbm_gb"], results[name]["loss"]))

    head = "VDNN_ALL" if "VDNN_ALL" in results else list(results)[0]
    base = results.get("BASELINE")
    # dominant kernel: the convolution class with the most device time over the timed steps of all
    # policies of this run (the same launches a kernel trace of this command sees, warm-up aside)
    prof = {}
    headline_bf16 = args.bf16 or all(is_bf16(n) for n in profiles)   # (a run of bfloat16 configurations only)
    for pname, p in profiles.items():
        if (args.bf16 or is_bf16(pname)) != headline_bf16:
            continue  # the roofline entry is taken over the runs of the headline element type
        for k, v in p.items():
            acc = prof.setdefault(k, {"launches": 0, "ms": 0.0, "flops": 0.0, "bytes": 0.0})
            for field in acc:
                acc[field] += v[field]
    conv = {k: v for k, v in prof.items() if k.startswith("conv_") and v["flops"] > 0}
    prof = {k: v for k, v in prof.items() if v["ms"] > 0}
    dom = max(conv, key=lambda k: conv[k]["ms"])
    d = conv[dom]
    achieved = d["flops"] / (d["ms"] * 1e-3) / 1e12
    peak = BF16_MFMA_PEAK_TFLOPS if "bf16mfma" in dom else FP32_MFMA_PEAK_TFLOPS
    conv_all_tf = sum(v["flops"] for v in conv.values()) / (sum(v["ms"] for v in conv.values()) * 1e-3) / 1e12
    kernels = {k: {"launches": v["launches"], "avg_ms": v["ms"] / max(v["launches"], 1),
                   "tflops": (v["flops"] / (v["ms"] * 1e-3) / 1e12) if v["flops"] else None,
                   "gbs": (v["bytes"] / (v["ms"] * 1e-3) / 1e9) if v["bytes"] else None}
               for k, v in sorted(prof.items(), key=lambda kv: -kv[1]["ms"])}
    out = {
        "metric": "VGG16-128 train img/s (VDNN_ALL vs BASELINE); peak HBM GB; conv MFMA util",
        "value": results[head]["images_per_s"], "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": results[head]["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16 (bf16 MFMA products, f32 accumulation, f32 master weights)" if headline_bf16 else "f32", "data": "synthetic (seeded N(0,1) inputs, integer labels, He-normal filters)",
        "config": {"workload": "VGG16 %s batch %d, one SGD step (fwd+bwd), policy %s, %s" % ("bf16-storage" if headline_bf16 else "fp32", args.batch, head, args.algo),
                   "batch": args.batch, "policy": head, "algo": args.algo},
        "policies": results,
        "vdnn_all_vs_baseline_speed": (results[head]["images_per_s"] / base["images_per_s"]) if base else None,
        "peak_hbm_reduction_vs_baseline": (base["peak_hbm_gb"] / results[head]["peak_hbm_gb"]) if base else None,
        "refined_vdnn_all_vs_baseline_speed": (results["VDNN_ALL+refined"]["images_per_s"] / base["images_per_s"])
        if base and "VDNN_ALL+refined" in results else None,
        "refined_peak_hbm_reduction_vs_baseline": (base["peak_hbm_gb"] / results["VDNN_ALL+refined"]["peak_hbm_gb"])
        if base and "VDNN_ALL+refined" in results else None,
        # fp32 VDNN_ALL with every value-preserving option on (refined lifetimes, fused rectifiers, compressed offload, packed
        # tensors kept in device memory): same losses as the literal `value` run, bit for bit
        "tuned_vdnn_all_vs_baseline_speed": (results["VDNN_ALL+refined+fused+zvc+keep"]["images_per_s"] / base["images_per_s"])
        if base and "VDNN_ALL+refined+fused+zvc+keep" in results else None,
        "tuned_peak_hbm_reduction_vs_baseline": (base["peak_hbm_gb"] / results["VDNN_ALL+refined+fused+zvc+keep"]["peak_hbm_gb"])
        if base and "VDNN_ALL+refined+fused+zvc+keep" in results else None,
        "losses_bit_identical": len({results[k]["loss"] for k in results if not is_bf16(k)}) <= 1
        and len({results[k]["loss"] for k in results if is_bf16(k)}) <= 1,
        "best_offloading_vs_fp32_baseline": best_offloading(results, base),
        # the same among the fp32 runs only: speed and memory against BASELINE with the reference's element type
        "best_fp32_offloading_vs_baseline": best_offloading({k: v for k, v in results.items() if not (args.bf16 or is_bf16(k))}, base),
        "conv_mfma_util": conv_all_tf / peak,
        "roofline": {"bound": "mfma", "kernel": dom, "achieved": achieved, "peak": peak, "unit": "TFLOP/s",
                     "frac": achieved / peak,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(dom) if args.batch == 128 and args.algo == "VDNN_MEMORY_OPT_ALGO" and not headline_bf16 else None,
                     "traffic_unit": "bytes per launch (L2 fetch + write-back, counters scaled by a known-size kernel)",
                     "algorithmic_flop_per_launch": d["flops"] / d["launches"],
                     "avg_launch_ms": d["ms"] / d["launches"], "launches": d["launches"]},
        "kernels": kernels,
        "step_mfma_frac": args.batch * FLOP_PER_IMAGE / (results[head]["ms_per_step"] * 1e-3) / 1e12 / peak,
    }
    if args.zvc_standalone:
        log("[bench] compacting kernels alone")
        out["zvc_standalone"] = zvc_standalone(be)
        log("[bench]   %s" % json.dumps(out["zvc_standalone"]))
    if not args.no_cpu_baseline:
        log("[bench] CPU baseline: checker, VGG16 batch %d" % args.cpu_batch)
        out["cpu_baseline"] = cpu_baseline(args.cpu_batch)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
