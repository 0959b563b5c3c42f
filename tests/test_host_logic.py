"""Host logic without a GPU: the C ABI library loads and exports every declared symbol, the pool
allocator, the policy setup, the prefetch scheduler and the allocation schedule replayed on a
plan-only context (no kernels run, nothing is computed), the seeded generator against the checker's.
"""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest

import oracle
import vdnn_implementation_amd.backend as be
from vdnn_implementation_amd import (ALEXNET, ALEXNET_LRN, BASELINE, OVERFEAT, VDNN_ALL, VDNN_CONV, VDNN_DYNAMIC_ALGO,
                                     VDNN_MEMORY_OPT_ALGO, VDNN_NONE, VDNN_PERF_OPT_ALGO, VGG16_64, VGG16_128, VGG16_256)
from vdnn_implementation_amd import enums
from vdnn_implementation_amd.backend import check, lib
from vdnn_implementation_amd.network import CAPI_SYMBOLS, Network, layer_spec, parse

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GB = 1e9


def declared_functions(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b(vdnn_[a-z0-9_]+)\s*\(", text))


def test_library_exports_every_declared_symbol():
    for header, table in (("vdnn_backend.h", be.BACKEND_SYMBOLS), ("vdnn_capi.h", CAPI_SYMBOLS)):
        names = declared_functions(header)
        assert names, header
        for n in names:
            assert hasattr(lib, n), "%s declares %s but the library does not export it" % (header, n)
        assert names == set(table), (names ^ set(table))


def test_enum_values_match_the_reference_header():
    # vdnn.h:23-61
    assert (BASELINE, VDNN_NONE, VDNN_ALL, VDNN_CONV) == (0, 1, 2, 3)
    assert (VDNN_MEMORY_OPT_ALGO, VDNN_PERF_OPT_ALGO, VDNN_DYNAMIC_ALGO) == (0, 1, 2)
    assert (enums.FC_GEMM, enums.CONV, enums.FC_CONV, enums.RELU, enums.SOFTMAX, enums.POOL) == (0, 1, 2, 3, 6, 7)
    assert (ALEXNET, OVERFEAT, VGG16_64, VGG16_128, VGG16_256) == (0, 1, 3, 4, 5)
    text = open(os.path.join(ROOT, "include", "vdnn.h")).read()
    for name, val in (("VDNN_CONV", 3), ("VDNN_DYNAMIC_ALGO", 2), ("POOL", 7), ("VGG16_256", 5), ("LRN", 10)):
        assert re.search(r"\b%s\s*=\s*%d\b" % (name, val), text)


def test_command_line_words():
    assert parse("VGG16_128", "VDNN_ALL", "VDNN_MEMORY_OPT_ALGO") == (VGG16_128, VDNN_ALL, VDNN_MEMORY_OPT_ALGO)
    assert parse("ALEXNET", "VDNN_NONE", "VDNN_PERF_OPT_ALGO") == (ALEXNET, VDNN_NONE, VDNN_PERF_OPT_ALGO)
    assert parse("OVERFEAT", "BASELINE", "VDNN_DYNAMIC_ALGO") == (OVERFEAT, BASELINE, VDNN_DYNAMIC_ALGO)
    with pytest.raises(ValueError):
        parse("RESNET", "BASELINE", "VDNN_MEMORY_OPT_ALGO")
    exe = os.path.join(ROOT, "vdnn_implementation_amd", "bin", "vdnn")
    out = subprocess.run([exe, "VGG16_64", "VDNN_CONV", "VDNN_MEMORY_OPT_ALGO", "--plan"], capture_output=True, text=True)
    assert out.returncode == 0 and "CNN Model Type: VGG16_64" in out.stdout and '"batch": 64' in out.stdout
    bad = subprocess.run([exe, "VGG16_64", "VDNN_SOME", "VDNN_MEMORY_OPT_ALGO", "--plan"], capture_output=True, text=True)
    assert bad.returncode != 0 and "VDNN type must be one of" in bad.stderr
    # the options of the recommended run: a budget, compressed offload, gradients written over inputs
    import json
    peaks = {}
    for extra in ([], ["--in-place"]):
        out = subprocess.run([exe, "VGG16_128", "VDNN_ALL", "VDNN_MEMORY_OPT_ALGO", "--plan", "--refined", "--fuse", "--zvc", "--offload-lag", "14",
                              "--prefetch-within-peak", "--packed-fraction", "0.6", "--hbm-budget-gb", "5.48"] + extra, capture_output=True, text=True)
        assert out.returncode == 0, out.stderr
        peaks[bool(extra)] = json.loads(out.stdout.strip().splitlines()[-1])
    assert not peaks[False]["plan_feasible"] and peaks[True]["plan_feasible"]
    assert peaks[True]["peak_bytes"] <= 5.48e9 < peaks[False]["peak_bytes"]


def test_command_line_reports_a_step_that_ran_out_of_memory():
    """Under an artificial cap a step that does not fit returns -1 (layer.h:110-128 of the reference); the program then
    prints no throughput and exits non-zero. A cap that the policy fits under runs as before."""
    import json
    exe = os.path.join(ROOT, "vdnn_implementation_amd", "bin", "vdnn")
    out = subprocess.run([exe, "VGG16_64", "VDNN_NONE", "VDNN_MEMORY_OPT_ALGO", "--plan", "--cap-gb", "4", "--warmup", "1"], capture_output=True, text=True)
    assert out.returncode == 3, (out.returncode, out.stderr)
    assert "forwardPropagation returned -1" in out.stderr and "warm-up step 0" in out.stderr
    last = json.loads(out.stdout.strip().splitlines()[-1])
    assert last["error"] == "out of memory" and "images_per_s" not in last and "Elapsed Time" not in out.stdout
    ok = subprocess.run([exe, "VGG16_64", "VDNN_ALL", "VDNN_MEMORY_OPT_ALGO", "--plan", "--cap-gb", "8"], capture_output=True, text=True)
    assert ok.returncode == 0 and json.loads(ok.stdout.strip().splitlines()[-1])["peak_bytes"] < 8e9
    # backward is where VDNN_ALL peaks (4.73 GB): a cap between the forward's need and that fails there
    mid = subprocess.run([exe, "VGG16_64", "VDNN_ALL", "VDNN_MEMORY_OPT_ALGO", "--plan", "--cap-gb", "4.5"], capture_output=True, text=True)
    assert mid.returncode == 3 and json.loads(mid.stdout.strip().splitlines()[-1])["failed_in"] in ("forward", "backward")


def test_reference_shaped_main_compiles_against_the_public_headers():
    """The class headers a caller of the reference includes (network.h, layer.h, vdnn.h) live under include/:
    a main of the shape of vdnn.cu:56-83 builds with the host compiler and -Iinclude alone, links against the
    library, and its VDNN_ALL schedule (replayed without a device) moves the bytes of the offload table."""
    import shutil
    import tempfile
    pkg = os.path.join(ROOT, "vdnn_implementation_amd")
    tmp = tempfile.mkdtemp(prefix="vdnn_main_")
    try:
        exe = os.path.join(tmp, "ref_main")
        cmd = ["g++", "-std=c++17", "-O1", "-I" + os.path.join(ROOT, "include"), os.path.join(ROOT, "tests", "cpp", "reference_shaped_main.cpp"),
               "-o", exe, "-L" + pkg, "-lvdnn_amd", "-Wl,-rpath," + pkg, "-Wl,-rpath-link,/opt/rocm/lib"]
        built = subprocess.run(cmd, capture_output=True, text=True)
        assert built.returncode == 0, built.stderr
        out = subprocess.run([exe, "VGG16_64", "VDNN_ALL", "VDNN_MEMORY_OPT_ALGO", "--plan"], capture_output=True, text=True)
        assert out.returncode == 0, out.stderr
        want = 14741667840 // 2  # the VGG16 batch 128 table at batch 64
        assert "status 0 0 layers 37 batch 64 input %d output 64000 offloaded %d prefetched %d dxdy %d" % (
            64 * 3 * 224 * 224, want, want, 64 * 64 * 224 * 224 * 4) in out.stdout, out.stdout
    finally:
        shutil.rmtree(tmp, ignore_errors=True)


def test_default_options_set_every_field():
    """A C caller declares the options on its stack: whatever the memory held, vdnn_network_default_options
    leaves every field (and the padding) at its default."""
    from vdnn_implementation_amd.network import Options
    o = Options()
    C.memset(C.byref(o), 0xFF, C.sizeof(o))
    lib.vdnn_network_default_options(C.byref(o))
    want = {"seed": 1, "prefetch_depth": 1, "plan_packed_fraction": 0.0}
    for name, _ in Options._fields_:
        assert getattr(o, name) == want.get(name, 0), name
    z = Options()
    lib.vdnn_network_default_options(C.byref(z))
    assert bytes(o) == bytes(z), "padding bytes differ"


# ---- pool allocator ---------------------------------------------------------------------------------
def test_pool_best_fit_coalescing_peak_and_cap():
    ctx = be.Context(plan_only=True, pool_bytes=256 << 20)
    base_free, total = ctx.pool_info()
    assert total == 256 << 20 and total - base_free == 64 << 20  # the staging area, taken at init
    a, b, c = ctx.alloc(1 << 20), ctx.alloc(3 << 20), ctx.alloc(1 << 20)
    assert ctx.pool_info()[0] == base_free - (5 << 20)
    assert a.ptr % 512 == 0 and b.ptr == a.ptr + (1 << 20) and c.ptr == b.ptr + (3 << 20)
    pb = b.ptr
    b.free()
    d = ctx.alloc(2 << 20)          # best fit: the 3 MiB hole, not the tail
    assert d.ptr == pb
    e = ctx.alloc(1 << 20)          # the remaining 1 MiB of the hole
    assert e.ptr == pb + (2 << 20)
    peak, extent = ctx.pool_peak()
    assert peak == (64 << 20) + (5 << 20)
    for x in (a, c, d, e):
        x.free()
    assert ctx.pool_info()[0] == base_free and ctx.live_blocks() == 1  # the staging area
    big = ctx.alloc(base_free)      # fully coalesced again
    big.free()
    with pytest.raises(be.OutOfMemory):
        ctx.alloc(base_free + 512)
    check(lib.vdnn_pool_set_cap(ctx.handle, (64 << 20) + (10 << 20)))
    x = ctx.alloc(8 << 20)
    with pytest.raises(be.OutOfMemory):
        ctx.alloc(4 << 20)
    x.free()
    assert lib.vdnn_pool_free(ctx.handle, C.c_void_p(12345)) == be.VDNN_EINVAL  # not a live block
    tiny = ctx.alloc(1)
    assert ctx.pool_info()[0] == base_free - 512  # 512-byte granularity
    tiny.free()
    ctx.close()


def test_pool_fragmentation_is_visible_in_the_extent():
    ctx = be.Context(plan_only=True, pool_bytes=128 << 20)
    blocks = [ctx.alloc(1 << 20) for _ in range(8)]
    for b in blocks[::2]:
        b.free()
    with_holes = ctx.alloc(2 << 20)  # no 2 MiB hole: goes to the tail
    assert with_holes.ptr > blocks[-1].ptr
    in_use, extent = ctx.pool_peak()
    assert extent >= in_use
    ctx.close()


# ---- policy setup (network.cu:875-940) and prefetch scheduler (network.cu:1198-1208) -----------------
def plan(cnn, policy, algo=VDNN_MEMORY_OPT_ALGO, batch=0, **kw):
    return Network(cnn, policy, algo, batch, plan_only=True, **kw)


def conv_layers(net):
    return [l for l, s in enumerate(net.specs) if s.type in (enums.FC_CONV, enums.CONV)]


@pytest.mark.parametrize("cnn,layers", [(ALEXNET, 19), (ALEXNET_LRN, 21), (OVERFEAT, 19), (VGG16_128, 37)])
def test_offload_sets(cnn, layers):
    for policy in (BASELINE, VDNN_NONE):
        with plan(cnn, policy, batch=2) as net:
            assert net.num_layers == layers
            assert not any(net.is_offloaded(l) for l in range(layers))
    with plan(cnn, VDNN_ALL, batch=2) as net:
        assert [net.is_offloaded(l) for l in range(layers)] == [True] * (layers - 1) + [False]
        pinned = sum(int(np.prod(net.src_shape(l))) * 4 for l in range(layers - 1))
        assert net.stats()["pinned_bytes"] == pinned
    with plan(cnn, VDNN_CONV, batch=2) as net:
        assert [l for l in range(layers) if net.is_offloaded(l)] == conv_layers(net)


def step(net):
    assert net.forwardPropagation() == 0
    assert net.backwardPropagation() == 0


def test_prefetch_sequences():
    # derived by replaying network.cu:1198-1208 on the reference's tables
    with plan(VGG16_128, VDNN_ALL, batch=1) as net:
        step(net)
        assert net.prefetch_trace() == [(l, l - 1) for l in range(36, 0, -1)]
    with plan(VGG16_128, VDNN_CONV, batch=1) as net:
        step(net)
        assert net.prefetch_trace() == [(36, 28), (28, 26), (26, 24), (24, 21), (21, 19), (19, 17), (17, 14), (14, 12),
                                        (12, 10), (10, 7), (7, 5), (5, 2), (2, 0)]
    with plan(ALEXNET, VDNN_CONV, batch=1) as net:
        step(net)
        assert net.prefetch_trace() == [(18, 10), (10, 8), (8, 6), (6, 3), (3, 0)]
    with plan(OVERFEAT, VDNN_CONV, batch=1) as net:
        step(net)
        assert net.prefetch_trace() == [(18, 17), (17, 15), (15, 13), (13, 10), (10, 8), (8, 6), (6, 3), (3, 0)]
    for cnn in (ALEXNET, OVERFEAT, ALEXNET_LRN):
        with plan(cnn, VDNN_ALL, batch=1) as net:
            step(net)
            L = net.num_layers
            assert net.prefetch_trace() == [(l, l - 1) for l in range(L - 1, 0, -1)]
    with plan(VGG16_128, VDNN_NONE, batch=1) as net:
        step(net)
        assert net.prefetch_trace() == []


STAGING = 64 << 20  # reduction staging area, taken from the pool at start


def test_peak_memory_of_the_literal_schedule_vgg16_128():
    """Replay of the reference's allocation schedule, 4-byte elements, no convolution workspace:
    BASELINE 18.58 GB, VDNN_NONE 15.38, VDNN_CONV 11.11, VDNN_ALL 8.85 (weights 0.553 GB included).
    The figures below add the 64 MiB staging area and 512-byte rounding; VDNN_ALL is 77 MB lower
    because the input block is released after its offload instead of being leaked."""
    want = {BASELINE: 18.58, VDNN_NONE: 15.38, VDNN_CONV: 11.11, VDNN_ALL: 8.85}
    got = {}
    for policy in want:
        with plan(VGG16_128, policy) as net:
            assert net.batch == 128
            step(net)
            got[policy] = net.stats()
            peak = (got[policy]["peak_bytes_in_use"] - STAGING) / GB
            assert abs(peak - want[policy]) < 0.09, (policy, peak)
            step(net)  # a second step must not grow the pool: nothing leaks
            assert net.stats()["peak_bytes_in_use"] == got[policy]["peak_bytes_in_use"]
    assert got[VDNN_ALL]["offload_bytes"] == got[VDNN_ALL]["prefetch_bytes"] == 14741667840
    assert abs(got[VDNN_CONV]["offload_bytes"] / GB - 4.65) < 0.01
    assert got[VDNN_CONV]["offload_bytes"] == got[VDNN_CONV]["prefetch_bytes"]
    assert got[BASELINE]["peak_bytes_in_use"] / got[VDNN_ALL]["peak_bytes_in_use"] > 2.09
    assert abs(got[BASELINE]["weight_bytes"] / GB - 0.553) < 0.001


def test_refined_lifetimes_cut_peak_memory_threefold():
    """ReLU inputs are dead after forward (their backward needs only y), convolution / FC / pooling
    outputs are released before their backward, ReLU backward runs in place. VGG16 batch 128:
    VDNN_ALL 8.84 -> 5.97 GB (3.1x below BASELINE) while the offload set shrinks from 14.74 to 7.80 GB."""
    with plan(VGG16_128, BASELINE) as net:
        step(net)
        base = net.stats()["peak_bytes_in_use"]
    want = {VDNN_NONE: (8.47, 0.0), VDNN_CONV: (5.97, 4.65), VDNN_ALL: (5.97, 7.80)}
    for policy, (peak_gb, offload_gb) in want.items():
        with plan(VGG16_128, policy, refined=True) as net:
            n0 = C.c_size_t()
            lib.vdnn_pool_live_blocks(net.context, C.byref(n0))
            step(net)
            step(net)
            st = net.stats()
            n1 = C.c_size_t()
            lib.vdnn_pool_live_blocks(net.context, C.byref(n1))
            assert n1.value == n0.value  # nothing leaks, nothing is freed twice
            assert abs(st["peak_bytes_in_use"] / GB - peak_gb) < 0.01
            assert abs(st["offload_bytes"] / GB - offload_gb) < 0.01 and st["offload_bytes"] == st["prefetch_bytes"]
            relu = [l for l, s in enumerate(net.specs) if s.type == enums.RELU]
            assert not any(net.is_offloaded(l) for l in relu)
    assert base / (5.97 * GB) > 3.0
    with plan(VGG16_128, BASELINE, refined=True) as net:  # BASELINE is never touched
        step(net)
        assert net.stats()["peak_bytes_in_use"] == base


def test_bf16_storage_halves_activations_and_offload_vgg16_512_under_48gb():
    """VGG16 batch 512 with bfloat16 activations under a 48 GB limit on bytes in use. By the reference's
    own allocation rule BASELINE needs 72.7 GB in float but 36.7 GB with 2-byte activations, so it
    fits under 48 GB; a limit it cannot meet is shown with 24 GB, where VDNN_NONE's forward returns -1 in
    dynamic mode and VDNN_ALL still fits. VDNN_ALL moves half the bytes of the float run."""
    cap = 48 * GB
    with plan(enums.VGG16_512, BASELINE, bf16=True, cap_bytes=cap, pool_bytes=120 * GB) as net:
        assert net.batch == 512
        assert net.forwardPropagation(True) == 0 and net.backwardPropagation(True) == 0
        base = net.stats()["peak_bytes_in_use"]
        assert abs(base / GB - 36.7) < 0.3
    with plan(enums.VGG16_512, BASELINE, pool_bytes=120 * GB) as net:  # float activations: 72.7 GB, over the limit
        step(net)
        assert abs(net.stats()["peak_bytes_in_use"] / GB - 72.7) < 0.3
    # BASELINE takes its buffers when it is built (network.cu:897-904), where a failed request is fatal as in
    # the reference; the policy that allocates per layer shows the clean failure under the same 24 GB limit
    with plan(enums.VGG16_512, VDNN_NONE, bf16=True, cap_bytes=24 * GB, pool_bytes=120 * GB) as net:
        assert net.forwardPropagation(True) == -1
    assert base > 24 * GB
    with plan(enums.VGG16_512, VDNN_ALL, bf16=True, cap_bytes=cap, pool_bytes=120 * GB) as net:
        assert net.forwardPropagation(True) == 0 and net.backwardPropagation(True) == 0
        st = net.stats()
        assert st["offload_bytes"] == st["prefetch_bytes"] == 14741667840 * 4 // 2  # batch x4, 2-byte elements
        assert st["peak_bytes_in_use"] < 24 * GB
        assert abs(st["weight_bytes"] / GB - 0.553) < 0.001  # float master parameters
    with plan(enums.VGG16_512, VDNN_ALL, bf16=True, cap_bytes=24 * GB, pool_bytes=120 * GB) as net:
        assert net.forwardPropagation(True) == 0 and net.backwardPropagation(True) == 0
    with plan(VGG16_128, VDNN_ALL) as f32, plan(VGG16_128, VDNN_ALL, bf16=True) as b16:
        step(f32)
        step(b16)
        acts32 = f32.stats()["peak_bytes_in_use"] - f32.stats()["weight_bytes"] - STAGING
        acts16 = b16.stats()["peak_bytes_in_use"] - b16.stats()["weight_bytes"] - STAGING
        assert abs(acts16 / acts32 - 0.5) < 0.01


def test_scheduling_slack_moves_the_same_bytes_and_leaks_nothing():
    """offloadLag / prefetchDepth change lifetimes only: same offload set, every block returned, and the
    extra memory is bounded and reproducible (VGG16 batch 128, refined VDNN_CONV: 5.96 GB up to a lag of four
    layers, 6.79 GB at six, 8.46 GB when nothing is recycled before the end of forward)."""
    with plan(VGG16_128, VDNN_CONV, refined=True) as net:
        step(net)
        ref = net.stats()
    for lag, depth, peak_gb in ((4, 1, 5.96), (6, 2, 6.79), (40, 3, 8.46)):
        with plan(VGG16_128, VDNN_CONV, refined=True, offload_lag=lag, prefetch_depth=depth) as net:
            n0 = C.c_size_t()
            lib.vdnn_pool_live_blocks(net.context, C.byref(n0))
            step(net)
            step(net)
            st = net.stats()
            n1 = C.c_size_t()
            lib.vdnn_pool_live_blocks(net.context, C.byref(n1))
            assert n1.value == n0.value
            assert st["offload_bytes"] == st["prefetch_bytes"] == ref["offload_bytes"]
            assert abs(st["peak_bytes_in_use"] / GB - peak_gb) < 0.02
            fetched = [p for _, p in net.prefetch_trace()]
            assert sorted(fetched, reverse=True) == fetched and len(set(fetched)) == len(fetched)  # top down, once each
    with plan(VGG16_128, VDNN_ALL, offload_lag=2, prefetch_depth=4) as net:
        step(net)
        assert [p for _, p in net.prefetch_trace()] == list(range(35, -1, -1))


def test_prefetch_depth_counts_packed_streams_on_their_way_back():
    """prefetchDepth bounds the tensors held ahead of their backward, whether they come back whole or as packed streams
    through the copy engine: at every fetch, the fetched tensors of layers still below the issuing layer (the new one
    included) number at most prefetchDepth, and the sequence is the same top-down order with and without compression."""
    traces = {}
    for compress in (False, True):
        for depth in (1, 2, 3):
            with plan(VGG16_128, VDNN_ALL, refined=True, fuse=True, compress=compress, offload_lag=6, prefetch_depth=depth) as net:
                step(net)
                trace = net.prefetch_trace()
                st = net.stats()
            fetched = [p for _, p in trace]
            assert sorted(fetched, reverse=True) == fetched and len(set(fetched)) == len(fetched)
            assert st["offload_bytes"] == st["prefetch_bytes"] > 0
            held_most = 0
            for i, (issuer, ident) in enumerate(trace):
                if issuer == ident:
                    continue   # a layer that expands or fetches its own input at the start of its backward holds nothing ahead
                held = [p for j, p in trace[:i + 1] if p < issuer and j != p]
                held_most = max(held_most, len(held))
                # (depth 1 is the reference's scan, network.cu:1198-1208: every layer's backward fetches the next tensor
                # down, also a layer whose own input was fetched by the layer above; the bound holds from depth 2 on)
                assert depth == 1 or len(held) <= depth, (compress, depth, issuer, held)
            assert depth == 1 or held_most == depth, (compress, depth, held_most)
            traces[compress, depth] = trace
    for depth in (1, 2, 3):
        assert [p for _, p in traces[True, depth]] == [p for _, p in traces[False, depth]]
        assert traces[True, depth] == traces[False, depth]


def test_plan_link_bytes_sends_tensors_over_the_link_before_packing_any():
    """planLinkBytes is an allowance of bytes per step and direction that a budget's plan spends on the link first: the
    members that must leave go over the link while their (packed) bytes fit it, and only then wait packed on the
    device. Same budget, same feasibility; fewer tensors packed; the bytes planned for the link within the allowance."""
    with plan(VGG16_128, BASELINE, batch=256) as r:
        step(r)
        base = r.stats()["peak_bytes_in_use"]
    kw = dict(refined=True, fuse=True, compress=True, in_place=True, recompute_first=True, offload_lag=-1, prefetch_within_peak=True,
              plan_packed_fraction=0.6, hbm_budget_bytes=int(base / 4.4))
    seen = {}
    for allowance in (0, int(2.5e9), int(3.5e9)):
        with plan(VGG16_128, VDNN_ALL, batch=256, plan_link_bytes=allowance, **kw) as net:
            step(net)
            step(net)
            places = net.placement()
            over = [l for l, p in enumerate(places) if p == 3]
            planned = sum(0.6 * 4 * net.specs[l].n * net.specs[l].c * net.specs[l].h * net.specs[l].w for l in over)
            assert net.plan_feasible() and net.stats()["peak_bytes_in_use"] <= kw["hbm_budget_bytes"]
            seen[allowance] = (over, places.count(2))
            if allowance:
                assert planned <= allowance
    assert seen[0][0] == [4] and seen[int(2.5e9)][0] == [4, 5] and seen[int(3.5e9)][0] == [4, 7]
    assert seen[0][1] > seen[int(2.5e9)][1] > seen[int(3.5e9)][1] == 0


def test_unfused_optimizer_costs_one_more_copy_of_the_parameters():
    for policy in (BASELINE, VDNN_ALL):
        with plan(VGG16_128, policy) as net:
            step(net)
            fused = net.stats()
        with plan(VGG16_128, policy, unfused_optimizer=True) as net:
            n0 = C.c_size_t()
            lib.vdnn_pool_live_blocks(net.context, C.byref(n0))
            step(net)
            st = net.stats()
            n1 = C.c_size_t()
            lib.vdnn_pool_live_blocks(net.context, C.byref(n1))
            assert n1.value == n0.value
        extra = st["peak_bytes_in_use"] - fused["peak_bytes_in_use"]
        assert abs(extra - fused["weight_bytes"]) < 64 * 512  # 32 parameter blocks, 512-byte granularity


def test_workspace_sizes_of_the_algorithm_modes_vgg16_128():
    """The workspace protocol of `layer.cu:268-294` (sizes asked per pass) for VGG16's layer shapes at batch 128: none in
    the memory-optimal mode; in the perf-optimal mode the size of the filter for forward and backward data wherever the
    reduced channels come in sixteens (the filter as two bfloat16 parts), and - with its Winograd variant selected - the
    transformed filter plus a chunk's transformed tensors on the layers Winograd takes. Host arithmetic only."""
    shapes = [(3, 64, 224), (64, 64, 224), (64, 128, 112), (128, 128, 112), (128, 256, 56), (256, 256, 56), (256, 512, 28),
              (512, 512, 28), (512, 512, 14)]
    assert lib.vdnn_conv_perf_variant(-1) == 0      # (an unknown value changes nothing and reports the current one)
    try:
        for c, k, hw in shapes:
            g = be.shape(128, c, hw, hw, k, 3, 3, 1, 1, 1, 1)
            filt = k * c * 9 * 4
            assert [int(lib.vdnn_conv_workspace_bytes(g, 0, p)) for p in range(3)] == [0, 0, 0]
            lib.vdnn_conv_perf_variant(0)
            split = [int(lib.vdnn_conv_workspace_bytes(g, 1, p)) for p in range(3)]
            assert split[:2] == ([0, 0] if c == 3 else [filt, filt])
            assert lib.vdnn_conv_perf_variant(1) == 0
            wino = [int(lib.vdnn_conv_workspace_bytes(g, 1, p)) for p in range(3)]
            assert lib.vdnn_conv_perf_variant(0) == 1
            if c >= 128:
                # transformed filter (36 values per tap set) and at least one sample's transformed input and output
                tiles = ((hw + 3) // 4) ** 2
                for p in range(2):
                    assert wino[p] >= 36 * k * c * 4 + 36 * (c + k) * tiles * 4 and wino[p] % 256 == 0
                assert wino[2] >= 36 * k * c * 4
                # backward filter of the split variant: more staging for its splits, or (14 x 14) Winograd's
                assert split[2] == 0 or split[2] >= filt
                if hw == 14:
                    assert split[2] == wino[2]
            else:
                assert wino == split
            # bfloat16 activations: the re-laid-out filter, whatever the variant
            assert int(lib.vdnn_conv_workspace_bytes_dtype(g, 1, 0, 1)) == (0 if c == 3 else filt)
    finally:
        lib.vdnn_conv_perf_variant(0)


def test_peak_memory_other_configs():
    for cnn, batch, base, allp in ((VGG16_64, 0, 9.57, 4.70), (OVERFEAT, 128, 1.90, 1.37), (ALEXNET, 32, 0.53, 0.44)):
        with plan(cnn, BASELINE, batch=batch) as net:
            step(net)
            assert abs((net.stats()["peak_bytes_in_use"] - STAGING) / GB - base) < 0.03
        with plan(cnn, VDNN_ALL, batch=batch) as net:
            step(net)
            # lower than the literal replay by one input block (released after its offload, not leaked)
            input_gb = net.getInputSize() * 4 / GB
            assert abs((net.stats()["peak_bytes_in_use"] - STAGING) / GB - (allp - input_gb)) < 0.012


def test_byte_counts_do_not_overflow_at_batch_256():
    # the reference's int byte math overflows here (network.cu:1010-1023, layer.h:240)
    with plan(VGG16_256, BASELINE) as net:
        assert net.batch == 256
        assert net.findMaxDxDySize() == 256 * 64 * 224 * 224 * 4 > 2 ** 31
        step(net)


def test_blocks_are_all_returned():
    for policy in (VDNN_NONE, VDNN_CONV, VDNN_ALL):
        with plan(ALEXNET_LRN, policy, batch=4) as net:
            ctxh = net.context
            n0 = C.c_size_t()
            lib.vdnn_pool_live_blocks(ctxh, C.byref(n0))
            for _ in range(3):
                step(net)
            n1 = C.c_size_t()
            lib.vdnn_pool_live_blocks(ctxh, C.byref(n1))
            assert n1.value == n0.value


def test_cap_makes_baseline_fail_cleanly_where_vdnn_all_fits():
    """The out-of-memory path of layer.h:110-128: in dynamic mode a failed pool request travels up as
    -1 through Layer::forward and forwardPropagation."""
    with plan(VGG16_64, VDNN_ALL) as net:
        step(net)
        need_all = net.stats()["peak_bytes_in_use"]
    cap = int(need_all * 1.05)
    with plan(VGG16_64, VDNN_ALL, cap_bytes=cap) as net:
        assert net.forwardPropagation(True) == 0 and net.backwardPropagation(True) == 0
    with plan(VGG16_64, VDNN_NONE, cap_bytes=cap) as net:
        assert net.forwardPropagation(True) == -1


def test_dynamic_algo_ladder():
    # network.cu:946-1008: with room to spare the first rung that fits is (VDNN_NONE, PERF_OPT)
    with plan(ALEXNET, BASELINE, VDNN_DYNAMIC_ALGO, batch=8) as net:
        assert (net.policy, net.algo) == (VDNN_NONE, VDNN_PERF_OPT_ALGO)
    with plan(VGG16_64, VDNN_ALL) as net:
        step(net)
        need_all = net.stats()["peak_bytes_in_use"]
    with plan(VGG16_64, VDNN_CONV, VDNN_PERF_OPT_ALGO) as net:  # the rung runs the workspace-using kernels
        step(net)
        need_conv = net.stats()["peak_bytes_in_use"]
    # room for VDNN_CONV but not VDNN_NONE
    with plan(VGG16_64, BASELINE, VDNN_DYNAMIC_ALGO, cap_bytes=int(need_conv * 1.02)) as net:
        assert (net.policy, net.algo) == (VDNN_CONV, VDNN_PERF_OPT_ALGO)
    with plan(VGG16_64, BASELINE, VDNN_DYNAMIC_ALGO, cap_bytes=int(need_all * 1.02)) as net:
        assert net.policy == VDNN_ALL


def test_dynamic_ladder_rebuilds_cleanly_after_trials_that_fail_half_way():
    """A trial step of the ladder that runs out of memory in the middle of forward leaves blocks, packed streams
    kept on the device and pending offloads behind; reset() forgets them with the pool they came from, so the
    configuration the ladder settles on steps without touching a block of the destroyed pool, and nothing leaks.
    A replay network built inside the constructor (prefetch_within_peak) does not change the outer one."""
    kw = dict(refined=True, fuse=True, compress=True, keep_packed=True, prefetch_within_peak=True, plan_packed_fraction=0.6)
    with plan(VGG16_64, VDNN_ALL, VDNN_PERF_OPT_ALGO, **kw) as net:
        step(net)
        need_all = net.stats()["peak_bytes_in_use"]
    with plan(VGG16_64, VDNN_NONE, VDNN_PERF_OPT_ALGO, **kw) as net:
        step(net)
        need_none = net.stats()["peak_bytes_in_use"]
    assert need_all < need_none
    for cap, want in ((int(need_none * 1.02), VDNN_NONE), (int(need_all * 1.02), VDNN_ALL)):
        with plan(VGG16_64, BASELINE, VDNN_DYNAMIC_ALGO, cap_bytes=cap, **kw) as net:
            assert net.policy == want
            n0 = live_blocks(net)
            for _ in range(2):
                assert net.forwardPropagation(True) == 0 and net.backwardPropagation(True) == 0
            assert live_blocks(net) == n0
            assert net.stats()["peak_bytes_in_use"] <= cap
    # the same with a forward that stops half-way outside the ladder: the next network in the process is unaffected
    with plan(VGG16_64, VDNN_NONE, cap_bytes=int(need_all), **kw) as net:
        assert net.forwardPropagation(True) == -1
    with plan(VGG16_64, VDNN_ALL, VDNN_PERF_OPT_ALGO, **kw) as net:
        step(net)
        assert net.stats()["peak_bytes_in_use"] == need_all


def test_dynamic_ladder_tries_its_last_rung():
    """network.cu:89-98 ends with a per-layer choice of algorithm, each workspace tried against an empty pool
    (layer.cu:1091-1147). Between the peaks of (VDNN_ALL, memory-optimal) and (VDNN_ALL, perf-optimal) that choice
    takes workspaces that no longer fit once the activations are there; the ladder tries the step and sends layers
    back to the memory-optimal kernels until it fits, so whatever it settles on steps within the cap."""
    for kw in ({}, dict(refined=True, fuse=True, in_place=True, recompute_first=True, offload_lag=4)):
        with plan(VGG16_64, VDNN_ALL, **kw) as net:
            step(net)
            lo = net.stats()["peak_bytes_in_use"]
        with plan(VGG16_64, VDNN_ALL, VDNN_PERF_OPT_ALGO, **kw) as net:
            step(net)
            hi = net.stats()["peak_bytes_in_use"]
        assert lo < hi
        for f in (0.02, 0.3, 0.6, 0.9, 0.995):
            cap = int(lo + (hi - lo) * f)
            with plan(VGG16_64, BASELINE, VDNN_DYNAMIC_ALGO, cap_bytes=cap, **kw) as net:
                assert net.policy == VDNN_ALL
                for _ in range(2):
                    assert net.forwardPropagation(True) == 0 and net.backwardPropagation(True) == 0
                assert net.stats()["peak_bytes_in_use"] <= cap


def test_custom_table_shape_inference_and_sanity():
    layers = [layer_spec(enums.FC_CONV, 2, 3, 20, 20, 1, 1, 8, 3), layer_spec(enums.RELU, 2, 8, 20, 20),
              layer_spec(enums.POOL, 2, 8, 20, 20, 0, 2, 0, 2), layer_spec(enums.FC_GEMM, 2, 800, 1, 1, 0, 0, 10, 1),
              layer_spec(enums.SOFTMAX, 2, 10, 1, 1)]
    with Network(layers=layers, policy=VDNN_ALL, plan_only=True) as net:
        assert net.dst_shape(0) == (2, 8, 20, 20) and net.dst_shape(2) == (2, 8, 10, 10) and net.dst_shape(3) == (2, 10, 1, 1)
        step(net)
        assert net.prefetch_trace() == [(4, 3), (3, 2), (2, 1), (1, 0)]


# ---- seeded generator: the host code's draw equals the checker's, bit for bit ------------------------
def test_seeded_generator_matches_the_checker():
    for seed, stream, std in ((1, 1, 1.0), (77, 100, 0.0589), (2 ** 40 + 3, 136, 0.0147)):
        a = np.empty(50000, np.float32)
        lib.vdnn_seeded_fill_normal(a.ctypes.data_as(C.POINTER(C.c_float)), a.size, seed, stream, 0.0, std)
        assert np.array_equal(a.view(np.uint32), oracle.fill_normal(a.size, seed, stream, 0.0, std).view(np.uint32))
    lab = np.empty(1000, np.int32)
    lib.vdnn_seeded_fill_labels(lab.ctypes.data_as(C.POINTER(C.c_int32)), lab.size, 9, 2, 1000)
    assert np.array_equal(lab, oracle.fill_labels(1000, 9, 2, 1000))


def test_tables_agree_with_the_checker():
    for cnn in (ALEXNET, ALEXNET_LRN, OVERFEAT, VGG16_128):
        o = oracle.Net(cnn=cnn, batch=2)
        with plan(cnn, BASELINE, batch=2) as net:
            assert net.num_layers == o.num_layers
            for l in range(net.num_layers):
                assert net.specs[l].type == o.desc[l].type
                assert net.src_shape(l) == o.src_shape(l) and net.dst_shape(l) == o.dst_shape(l)
        o.close()


def test_fused_rectifiers_own_no_tensor_and_leak_nothing():
    """fuse: a ReLU behind a CONV / FC layer has no output block (its layer is elided), is never offloaded, and
    every policy still returns all blocks. VGG16 batch 128: BASELINE keeps 6.94 GB less (the 15 ReLU outputs),
    VDNN_ALL moves the bytes of the refined schedule (the ReLU inputs are not tensors of their own)."""
    with plan(VGG16_128, BASELINE) as net:
        step(net)
        base = net.stats()["peak_bytes_in_use"]
    with plan(VGG16_128, BASELINE, fuse=True) as net:
        step(net)
        relu_out = sum(int(np.prod(net.dst_shape(l))) * 4 for l, s in enumerate(net.specs) if s.type == enums.RELU)
        assert net.stats()["peak_bytes_in_use"] == base - relu_out
        assert abs(relu_out / GB - 6.94) < 0.01
    with plan(VGG16_128, VDNN_ALL, refined=True) as net:
        step(net)
        ref = net.stats()
    for policy, kw in ((VDNN_NONE, {}), (VDNN_CONV, {}), (VDNN_ALL, {}), (VDNN_ALL, {"refined": True}),
                       (VDNN_CONV, {"refined": True, "offload_lag": 6, "prefetch_depth": 2})):
        with plan(VGG16_128, policy, fuse=True, **kw) as net:
            n0 = C.c_size_t()
            lib.vdnn_pool_live_blocks(net.context, C.byref(n0))
            step(net)
            step(net)
            n1 = C.c_size_t()
            lib.vdnn_pool_live_blocks(net.context, C.byref(n1))
            assert n1.value == n0.value
            st = net.stats()
            assert not any(net.is_offloaded(l) for l, s in enumerate(net.specs) if s.type == enums.RELU)
            if policy == VDNN_ALL:
                assert st["offload_bytes"] == st["prefetch_bytes"] == ref["offload_bytes"]
                if kw.get("refined"):
                    assert st["peak_bytes_in_use"] <= ref["peak_bytes_in_use"]


def live_blocks(net):
    n = C.c_size_t()
    lib.vdnn_pool_live_blocks(net.context, C.byref(n))
    return n.value


def test_keep_tail_takes_the_deepest_members_out_of_the_offload_set():
    """keep_tail_bytes walks the policy's offload set from the last layer down and keeps what fits on the device."""
    with plan(VGG16_128, VDNN_CONV, batch=128) as net:
        convs = conv_layers(net)
        size = {l: int(np.prod(net.src_shape(l))) * 4 for l in convs}
    for keep in (0, 1, size[convs[-1]], size[convs[-1]] + size[convs[-2]] + 5, sum(size.values())):
        want, left = list(convs), keep
        while want and size[want[-1]] <= left:
            left -= size[want.pop()]
        with plan(VGG16_128, VDNN_CONV, batch=128, keep_tail_bytes=keep) as net:
            assert [l for l in range(net.num_layers) if net.is_offloaded(l)] == want, keep
            step(net)
            assert net.stats()["offload_bytes"] == sum(size[l] for l in want)
            assert net.stats()["prefetch_bytes"] == sum(size[l] for l in want)
    # the tail is small and gone before the large tensors come back: the peak of the plan does not move
    with plan(VGG16_128, VDNN_CONV, batch=128, refined=True) as a, \
         plan(VGG16_128, VDNN_CONV, batch=128, refined=True, keep_tail_bytes=int(1.2e9)) as b:
        step(a); step(b)
        assert len([l for l in range(b.num_layers) if b.is_offloaded(l)]) < len(conv_layers(a))
        assert b.stats()["peak_bytes_in_use"] == a.stats()["peak_bytes_in_use"]
        assert live_blocks(b) == live_blocks(a)


def test_compressed_offload_plans_for_the_longest_stream_and_leaks_nothing():
    """Planning has no data: it holds a staging block as long as the longest stream beside each packed tensor."""
    for policy, kw in ((VDNN_CONV, {}), (VDNN_ALL, {"refined": True, "offload_lag": 6, "prefetch_depth": 2}), (VDNN_ALL, {"fuse": True})):
        with plan(VGG16_128, policy, batch=16, **kw) as a, plan(VGG16_128, policy, batch=16, compress=True, **kw) as b:
            for _ in range(2):
                step(a); step(b)
            sa, sb = a.stats(), b.stats()
            assert sb["offload_bytes"] == sa["offload_bytes"] and sb["prefetch_bytes"] == sa["prefetch_bytes"]
            assert sa["pinned_bytes"] < sb["pinned_bytes"] < sa["pinned_bytes"] * 1.04
            assert sa["peak_bytes_in_use"] <= sb["peak_bytes_in_use"]
            assert live_blocks(b) == live_blocks(a)


def test_prefetch_within_peak_fetches_earlier_and_holds_the_peak():
    """The replay of the schedule tells backward where a tensor may come back early without raising the peak."""
    for policy, kw in ((VDNN_CONV, {}), (VDNN_CONV, {"refined": True, "offload_lag": 6}), (VDNN_ALL, {"refined": True}),
                       (VDNN_ALL, {"fuse": True, "offload_lag": 3, "prefetch_depth": 2}), (VDNN_CONV, {"refined": True, "keep_tail_bytes": int(1e9)})):
        with plan(VGG16_128, policy, batch=128, **kw) as a, plan(VGG16_128, policy, batch=128, prefetch_within_peak=True, **kw) as b:
            for _ in range(2):
                step(a); step(b)
            sa, sb = a.stats(), b.stats()
            assert sb["peak_bytes_in_use"] == sa["peak_bytes_in_use"], (policy, kw)
            assert sb["prefetch_bytes"] == sa["prefetch_bytes"] and sb["offload_bytes"] == sa["offload_bytes"]
            ta, tb = a.prefetch_trace(), b.prefetch_trace()
            assert [p for _, p in tb] == [p for _, p in ta], "the same tensors in the same order"
            assert all(lb >= la for (la, _), (lb, _) in zip(ta, tb)), "never later than the plain schedule"
            assert any(lb > la for (la, _), (lb, _) in zip(ta, tb)), "some of them earlier"
            assert live_blocks(b) == live_blocks(a)
    # BASELINE has nothing to fetch: the option is accepted and changes nothing
    with plan(VGG16_128, BASELINE, batch=128, prefetch_within_peak=True) as net:
        step(net)
        assert net.prefetch_trace() == []


def test_packed_tensors_kept_on_the_device_plan():
    """keep_packed: the packed stream of a rectified offloaded tensor stays in its staging block; nothing of it crosses
    the link, its own layer expands it at the start of its backward, and the peak follows the assumed stream length."""
    kw = dict(refined=True, fuse=True, compress=True)
    with plan(VGG16_128, VDNN_ALL, batch=128, **kw) as moved, \
         plan(VGG16_128, VDNN_ALL, batch=128, keep_packed=True, plan_packed_fraction=0.57, **kw) as kept, \
         plan(VGG16_128, VDNN_ALL, batch=128, keep_packed=True, **kw) as kept_worst:
        for net in (moved, kept, kept_worst):
            step(net); step(net)
        sm, sk, sw = moved.stats(), kept.stats(), kept_worst.stats()
        # only the tensors that are not rectified (the network input) still travel
        plain = [l for l in range(kept.num_layers) if kept.is_offloaded(l)]
        first = int(np.prod(kept.src_shape(0))) * 4
        assert sk["offload_bytes"] == first == sk["prefetch_bytes"] and 0 in plain
        assert sm["offload_bytes"] > 7e9
        # every kept tensor is expanded by its own layer; the one that travelled is fetched a layer ahead
        trace = kept.prefetch_trace()
        assert sorted(p for _, p in trace) == plain
        assert all(l == p for l, p in trace if p != 0) and (2, 0) in trace
        # at 0.57 of a tensor the step holds less than a third of BASELINE's 18.65 GB; at the longest stream it does not
        assert sk["peak_bytes_in_use"] < 18.65e9 / 3 < sw["peak_bytes_in_use"]
        assert live_blocks(kept) == live_blocks(moved) == live_blocks(kept_worst)


def test_hbm_budget_places_each_tensor_and_reports_the_floor():
    """hbm_budget_bytes: every member of the offload set stays on the device, waits there as a packed stream, or crosses
    the link - the cheapest that keeps a replay of the step within the budget. VGG16 batch 128, float, a packed stream
    taken as 0.57 of its tensor: a third of BASELINE's 18.65 GB needs no link at all, and below 5.63 GB no placement
    helps - that is convolution 1_2's backward (input, output gradient, input gradient: 3 x 1.64 GB, plus the
    parameters and the staging area), when nothing that could be moved is left on the device."""
    kw = dict(refined=True, fuse=True, compress=True, plan_packed_fraction=0.57)
    with plan(VGG16_128, BASELINE) as net:
        step(net)
        base = net.stats()["peak_bytes_in_use"]
    seen = {}
    for ratio in (2.0, 3.0, 3.3, 4.0):
        budget = int(base / ratio)
        with plan(VGG16_128, VDNN_ALL, hbm_budget_bytes=budget, **kw) as net:
            n0 = live_blocks(net)
            step(net); step(net)
            assert live_blocks(net) == n0
            st, places = net.stats(), net.placement()
            seen[ratio] = (net.plan_feasible(), net.plan_peak_bytes(), st, places)
            assert st["peak_bytes_in_use"] == net.plan_peak_bytes(), "the step holds what the plan's replay held"
            members = [l for l, p in enumerate(places) if p]
            assert members == [l for l, s in enumerate(net.specs[:-1]) if s.type != enums.RELU]   # fused, refined VDNN_ALL
            assert [l for l in members if places[l] in (2, 3)] == [l for l in range(net.num_layers) if net.is_offloaded(l)]
            link = sum(int(np.prod(net.src_shape(l))) * 4 for l in members if places[l] == 3)
            assert st["offload_bytes"] == st["prefetch_bytes"] == link
    assert seen[2.0][0] and set(seen[2.0][3]) == {0, 1}                       # fits as it is: nothing packed, nothing moved
    assert seen[3.0][0] and seen[3.0][1] <= base / 3 and 3 not in seen[3.0][3] and 2 in seen[3.0][3]
    assert seen[3.3][0] and abs(seen[3.3][1] / GB - 5.63) < 0.01 and 3 not in seen[3.3][3]
    assert not seen[4.0][0] and abs(seen[4.0][1] / GB - 5.63) < 0.01       # the floor: 3.31 x below BASELINE
    # more is packed as the budget shrinks, never less
    packed = {r: {l for l, p in enumerate(seen[r][3]) if p >= 2} for r in seen}
    assert packed[2.0] <= packed[3.0] <= packed[3.3] <= packed[4.0]
    # without packing the same budget sends the largest tensors over the link instead
    with plan(VGG16_128, VDNN_ALL, hbm_budget_bytes=int(base / 2.5), refined=True, fuse=True) as net:
        step(net)
        assert net.plan_feasible() and set(net.placement()) == {0, 1, 3}
        assert net.stats()["offload_bytes"] > 1.6e9
    # BASELINE and VDNN_NONE offload nothing: the budget is accepted and changes nothing
    with plan(VGG16_128, VDNN_NONE, hbm_budget_bytes=int(base / 3), **kw) as net:
        step(net)
        assert set(net.placement()) == {0} and net.stats()["offload_bytes"] == 0


def test_gradients_written_over_inputs_lower_the_floor():
    """in_place: a convolution above the first and a 2x2 pooling layer write their input gradient over their input where
    the layer below does not read that tensor again. VGG16 batch 128, float, fused rectifiers: convolution 1_2's backward
    then holds two tensors of 1.64 GB instead of three, and the floor of the placement moves from 5.63 GB to what
    convolution 1_2's *forward* holds - input, output and the input's packed stream on its way out: 4.93 GB, 3.79 x
    below BASELINE. Every block still goes back to the pool exactly once."""
    kw = dict(refined=True, fuse=True, compress=True, plan_packed_fraction=0.6)
    with plan(VGG16_128, BASELINE) as net:
        step(net)
        base = net.stats()["peak_bytes_in_use"]
    with plan(VGG16_128, VDNN_ALL, in_place=True, **kw) as net:
        over = [l for l in range(net.num_layers) if net.grad_over_src(l)]
        convs, pools = conv_layers(net), [l for l, s in enumerate(net.specs) if s.type == enums.POOL]
        assert over == sorted(convs[1:] + pools[:4])      # not the first convolution; the last pooling layer is 14 x 14: 7 columns
    with plan(VGG16_128, VDNN_ALL, in_place=True, refined=True) as net:   # separate ReLU layers read their output in backward
        assert [l for l in range(net.num_layers) if net.grad_over_src(l)] == [l for l in conv_layers(net)[1:] if net.specs[l - 1].type == enums.POOL]
    with plan(VGG16_128, VDNN_ALL, in_place=True) as net:                 # needs refined lifetimes
        assert not any(net.grad_over_src(l) for l in range(net.num_layers))
    with plan(VGG16_128, BASELINE, in_place=True, refined=True, fuse=True) as net:
        assert not any(net.grad_over_src(l) for l in range(net.num_layers))
    peaks = {}
    for in_place in (False, True):
        for name, extra in (("keep", dict(keep_packed=True)), ("floor", dict(hbm_budget_bytes=1, prefetch_within_peak=True)),
                            ("none", None)):
            opts = dict(kw, **extra) if extra is not None else dict(refined=True, fuse=True)
            with plan(VGG16_128, VDNN_NONE if extra is None else VDNN_ALL, in_place=in_place, **opts) as net:
                n0 = live_blocks(net)
                step(net); step(net)
                assert live_blocks(net) == n0
                peaks[name, in_place] = net.stats()["peak_bytes_in_use"]
                if name == "floor":
                    assert not net.plan_feasible() and net.plan_peak_bytes() == peaks[name, in_place]
    assert abs(peaks["floor", False] / GB - 5.63) < 0.01 and abs(peaks["floor", True] / GB - 4.93) < 0.01
    assert base / peaks["floor", True] > 3.78
    assert peaks["keep", True] < peaks["keep", False] and peaks["none", True] <= peaks["none", False]
    # other networks: same bookkeeping, overlapping pooling windows and LRN layers keep their gradients apart
    for cnn in (ALEXNET_LRN, OVERFEAT):
        with plan(cnn, VDNN_ALL, batch=16, in_place=True, refined=True, fuse=True) as net:
            n0 = live_blocks(net)
            step(net); step(net)
            assert live_blocks(net) == n0
            for l in range(net.num_layers):
                if net.grad_over_src(l):
                    assert l > 0 and net.specs[l].type in (enums.CONV, enums.FC_CONV, enums.POOL) and net.specs[l - 1].type != enums.LRN


def test_first_layer_computed_again_instead_of_kept():
    """recompute_first: the output of a first convolution over at most four channels is released behind its consumer's
    forward and computed again before the consumer's backward; the network input stays on the device for it. VGG16 batch
    128, float, with gradients written over inputs: every rectified tensor packed in HBM fits 4.61 GB - a quarter of
    BASELINE with nothing on the link - and the floor of the placement is convolution 1_2 with its input and its output
    alone: 3.99 GB, 4.68 x below BASELINE."""
    kw = dict(refined=True, fuse=True, compress=True, plan_packed_fraction=0.6, in_place=True)
    with plan(VGG16_128, BASELINE) as net:
        step(net)
        base = net.stats()["peak_bytes_in_use"]
    with plan(VGG16_128, VDNN_ALL, recompute_first=True, keep_packed=True, **kw) as net:
        assert net.recomputed_layer() == 2 and not net.is_offloaded(0) and not net.is_offloaded(2)
        n0 = live_blocks(net)
        step(net); step(net)
        assert live_blocks(net) == n0
        st = net.stats()
        assert abs(st["peak_bytes_in_use"] / GB - 4.61) < 0.01 and st["offload_bytes"] == 0 and base / st["peak_bytes_in_use"] > 4.0
    with plan(VGG16_128, VDNN_ALL, recompute_first=True, hbm_budget_bytes=int(base / 4), prefetch_within_peak=True, offload_lag=14, **kw) as net:
        step(net); step(net)
        assert net.plan_feasible() and 3 not in net.placement() and net.stats()["peak_bytes_in_use"] <= base / 4
    with plan(VGG16_128, VDNN_ALL, recompute_first=True, hbm_budget_bytes=1, prefetch_within_peak=True, **kw) as net:
        n0 = live_blocks(net)
        step(net); step(net)
        assert live_blocks(net) == n0
        assert not net.plan_feasible() and abs(net.plan_peak_bytes() / GB - 3.99) < 0.01
        assert net.placement()[4] == 3 and net.placement()[0] == net.placement()[2] == 0   # pool1's input over the link; nothing to place for layers 0 and 2
    # where it does not apply: no refined lifetimes, BASELINE, a first layer with many channels, a consumer behind a ReLU layer of its own
    with plan(VGG16_128, VDNN_ALL, recompute_first=True) as net:
        assert net.recomputed_layer() == -1
    with plan(VGG16_128, BASELINE, recompute_first=True, refined=True, fuse=True) as net:
        assert net.recomputed_layer() == -1
    with plan(VGG16_128, VDNN_ALL, recompute_first=True, refined=True) as net:
        assert net.recomputed_layer() == -1
        step(net)
    for cnn in (ALEXNET_LRN, OVERFEAT, ALEXNET):
        with plan(cnn, VDNN_ALL, batch=16, recompute_first=True, refined=True, fuse=True, in_place=True) as net:
            assert net.recomputed_layer() == 2
            n0 = live_blocks(net)
            step(net); step(net)
            assert live_blocks(net) == n0


def test_the_plan_chooses_the_offload_lag():
    """offload_lag < 0 with a budget: the lag is part of the plan. What waits for its copy counts against the budget for
    as long as the lag, so the longest lag is not always the one that fits with the fewest bytes on the link. VGG16 batch
    128 with gradients over inputs and the first layer computed again: down to BASELINE / 4.1 fourteen layers fit, at
    BASELINE / 4.2 eight, and below the floor the plan with the lowest peak stands."""
    kw = dict(refined=True, fuse=True, compress=True, plan_packed_fraction=0.6, in_place=True, recompute_first=True, prefetch_within_peak=True)
    with plan(VGG16_128, BASELINE) as net:
        step(net)
        base = net.stats()["peak_bytes_in_use"]
    seen = {}
    for ratio in (4.0, 4.1, 4.2, 4.5, 5.0):
        with plan(VGG16_128, VDNN_ALL, hbm_budget_bytes=int(base / ratio), offload_lag=-1, **kw) as net:
            n0 = live_blocks(net)
            step(net); step(net)
            assert live_blocks(net) == n0
            seen[ratio] = (net.offload_lag(), net.plan_feasible(), net.placement().count(3), net.stats()["peak_bytes_in_use"])
            assert net.stats()["peak_bytes_in_use"] == net.plan_peak_bytes()
            # the same plan with that lag spelt out
            with plan(VGG16_128, VDNN_ALL, hbm_budget_bytes=int(base / ratio), offload_lag=net.offload_lag(), **kw) as fixed:
                assert fixed.placement() == net.placement() and fixed.plan_peak_bytes() == net.plan_peak_bytes()
    assert seen[4.0][:3] == (14, True, 0) and seen[4.1][:3] == (14, True, 1) and seen[4.2][:3] == (8, True, 1)
    assert seen[4.5][1] and seen[4.5][0] < 8 and seen[4.5][2] == 1
    assert not seen[5.0][1] and abs(seen[5.0][3] / GB - 3.99) < 0.01
    for ratio in (4.0, 4.1, 4.2, 4.5):
        assert seen[ratio][3] <= base / ratio
    # without a budget a negative lag is no lag
    with plan(VGG16_128, VDNN_ALL, offload_lag=-1, refined=True) as a, plan(VGG16_128, VDNN_ALL, offload_lag=0, refined=True) as b:
        step(a); step(b)
        assert a.offload_lag() == 0 and a.stats() == b.stats()


def test_packed_streams_come_back_through_a_block_of_their_own_length():
    """A packed stream that crossed the link returns through the copy engine into a block sized from its length, a layer
    ahead of its backward; the layer itself expands it. What is held a layer ahead is the stream, not the tensor: the
    refined VDNN_ALL schedule of VGG16 batch 128 peaks lower than with plain copies, and moves the same tensors."""
    kw = dict(refined=True, fuse=True)
    with plan(VGG16_128, VDNN_ALL, **kw) as plain, plan(VGG16_128, VDNN_ALL, compress=True, plan_packed_fraction=0.57, **kw) as packed:
        for net in (plain, packed):
            n0 = live_blocks(net)
            step(net); step(net)
            assert live_blocks(net) == n0
        a, b = plain.stats(), packed.stats()
        assert b["offload_bytes"] == a["offload_bytes"] == b["prefetch_bytes"] == a["prefetch_bytes"]
        assert plain.prefetch_trace() == packed.prefetch_trace()   # the same tensors fetched by the same layers
        assert b["peak_bytes_in_use"] < a["peak_bytes_in_use"] - 0.25 * GB


def test_overlap_of_copies_and_kernels_from_intervals():
    """The interval arithmetic behind the bench's and the trace summary's overlap fraction, on a case worked by hand:
    kernels [0,10] and [12,20]; a device-to-host copy [5,15], a host-to-device copy [14,30]."""
    from vdnn_implementation_amd import trace_overlap as t
    s = t.summarize([("compute", 0, 10), ("compute", 12, 20), ("d2h", 5, 15), ("h2d", 14, 30), ("compute", 3, 4)])
    assert (s["span"], s["compute_busy"], s["copy_busy"], s["d2h_busy"], s["h2d_busy"]) == (30, 18, 25, 10, 16)
    assert s["copy_beside_compute"] == 13 and s["overlap_fraction"] == 13 / 25 and s["duplex"] == 1 and s["copy_exposed"] == 12
    assert t.summarize([("compute", 0, 5)])["overlap_fraction"] is None
    recs = [("conv_fwd_128x128", 0, 0.0, 2.0), ("offload_d2h", 1, 1.0, 4.0), ("offload_zvc_pack", 3, 0.5, 0.7), ("prefetch_h2d", 2, 3.0, 5.0),
            ("prefetch_zvc_device", 0, 5.0, 5.5)]
    assert sorted(t.from_profile(recs)) == [("compute", 0.0, 2.0), ("compute", 5.0, 5.5), ("d2h", 1.0, 4.0), ("h2d", 3.0, 5.0)]
