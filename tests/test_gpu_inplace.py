"""GPU parity of input gradients written over the layer's own input, through the C ABI.

The reference allocates a layer's gradData beside its srcData (layer.cu:599, 897, 999-1011). Where nothing reads the
input again, the kernels here may be handed dx == x: the result must be the bits of the call with a separate dx, and a
network that runs its backward that way must keep every bit of the BASELINE step while holding less memory.
"""
import numpy as np
import pytest

import oracle
import vdnn_implementation_amd.backend as be
from gpu_util import Dev, _workspace, announce
from test_gpu_fused import assert_fused_matches, relu
from test_gpu_network import assert_bit_identical, run_steps, small_specs
from test_gpu_zvc import rectified
from util import to_bf16_bits
from vdnn_implementation_amd import (ALEXNET_LRN, BASELINE, OVERFEAT, VDNN_ALL, VDNN_CONV, VDNN_MEMORY_OPT_ALGO, VDNN_NONE,
                                     VDNN_PERF_OPT_ALGO, VGG16_128)
from vdnn_implementation_amd.backend import check, lib
from vdnn_implementation_amd.network import Network

pytestmark = pytest.mark.gpu

IN_PLACE_GEOMS = [
    (2, 64, 14, 14, 64, 3, 3, 1, 1, 1, 1),      # few tiles: split reduction, the mask sits in the reduction kernel
    (8, 128, 28, 28, 128, 3, 3, 1, 1, 1, 1),    # many tiles: the mask sits in the tile kernel's epilogue
    (128, 512, 14, 14, 512, 3, 3, 1, 1, 1, 1),  # whole tiles plus a split last round
    (2, 48, 27, 27, 96, 5, 5, 2, 2, 1, 1),      # 5x5
    (2, 70, 9, 13, 130, 3, 3, 1, 1, 1, 1),      # nothing divides the tiles
    (3, 64, 32, 32, 64, 3, 3, 1, 1, 1, 1),      # the windowed kernel's shape in bfloat16
    (2, 96, 12, 12, 40, 1, 1, 0, 0, 1, 1),      # 1x1
]
NOT_IN_PLACE_GEOMS = [
    (1, 16, 20, 24, 32, 3, 5, 1, 2, 2, 1),      # strided
    (5, 64, 6, 6, 200, 6, 6, 0, 0, 1, 1),       # window = input: one dense product
    (2, 3, 32, 32, 16, 3, 3, 1, 1, 1, 1),       # three input channels
]


@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
@pytest.mark.parametrize("algo", [0, 1])
@pytest.mark.parametrize("geom", IN_PLACE_GEOMS, ids=lambda g: "x".join(map(str, g)))
def test_backward_data_over_its_input(geom, algo, bf16):
    g = be.shape(*geom)
    assert lib.vdnn_conv_bwd_data_in_place_ok(g) == 1
    rng = np.random.default_rng(hash(geom) % (2 ** 31) + 11)
    x = relu(rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32))
    P, Q = lib.vdnn_out_dim(g.h, g.pad_h, g.r, g.stride_h), lib.vdnn_out_dim(g.w, g.pad_w, g.s, g.stride_w)
    dy = rng.standard_normal((g.n, g.k, P, Q)).astype(np.float32)
    w = (rng.standard_normal((g.k, g.c, g.r, g.s)) * np.sqrt(2.0 / (g.c * g.r * g.s))).astype(np.float32)
    ctx = be.Context(pool_bytes=2 << 30)
    try:
        if bf16:
            check(lib.vdnn_ctx_set_activation_dtype(ctx.handle, 1))
            x, dy = oracle.round_bf16(x), oracle.round_bf16(dy)
        dt = np.uint16 if bf16 else np.float32
        enc = (lambda a: to_bf16_bits(a)) if bf16 else (lambda a: a)
        announce("backward data over its input", geom, "algo", algo, "bf16" if bf16 else "f32")
        with Dev(ctx) as d:
            a, bw = d.up(enc(dy), dt), d.up(w)
            gate, over = d.up(enc(x), dt), d.up(enc(x), dt)
            apart, plain_over = d.empty(x.shape, dt), d.up(enc(x), dt)
            ws, nws = _workspace(d, g, algo, 1)
            check(lib.vdnn_conv_bwd_data_relu(ctx.handle, None, g, algo, a.ptr, bw.ptr, gate.ptr, apart.ptr, ws, nws))
            check(lib.vdnn_conv_bwd_data_relu(ctx.handle, None, g, algo, a.ptr, bw.ptr, over.ptr, over.ptr, ws, nws))
            want, got = apart.download(x.shape, dt), over.download(x.shape, dt)
            assert np.array_equal(got, want), "masked gradient written over the input that masks it"
            # without the mask the kernel never reads the input: any tensor may receive the gradient
            check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, algo, a.ptr, bw.ptr, apart.ptr, ws, nws))
            check(lib.vdnn_conv_bwd_data(ctx.handle, None, g, algo, a.ptr, bw.ptr, plain_over.ptr, ws, nws))
            assert np.array_equal(plain_over.download(x.shape, dt), apart.download(x.shape, dt))
    finally:
        ctx.close()


@pytest.mark.parametrize("geom", NOT_IN_PLACE_GEOMS, ids=lambda g: "x".join(map(str, g)))
def test_shapes_that_cannot_write_over_their_input_say_so(geom):
    g = be.shape(*geom)
    assert lib.vdnn_conv_bwd_data_in_place_ok(g) == 0
    rng = np.random.default_rng(5)
    x = relu(rng.standard_normal((g.n, g.c, g.h, g.w)).astype(np.float32))
    P, Q = lib.vdnn_out_dim(g.h, g.pad_h, g.r, g.stride_h), lib.vdnn_out_dim(g.w, g.pad_w, g.s, g.stride_w)
    dy = rng.standard_normal((g.n, g.k, P, Q)).astype(np.float32)
    w = rng.standard_normal((g.k, g.c, g.r, g.s)).astype(np.float32)
    ctx = be.Context(pool_bytes=1 << 30)
    try:
        announce("backward data over its input refused", geom)
        with Dev(ctx) as d:
            a, bw, over = d.up(dy), d.up(w), d.up(x)
            assert lib.vdnn_conv_bwd_data_relu(ctx.handle, None, g, 0, a.ptr, bw.ptr, over.ptr, over.ptr, None, 0) != 0
            assert np.array_equal(over.download(x.shape), x), "a refused call touches nothing"
    finally:
        ctx.close()


@pytest.mark.parametrize("bf16", [False, True], ids=["f32", "bf16"])
@pytest.mark.parametrize("n,c,h,w", [(2, 8, 16, 16), (3, 5, 6, 20), (1, 3, 224, 224)])
def test_maxpool_backward_over_its_input(n, c, h, w, bf16):
    g = be.shape(n, c, h, w, 0, 2, 2, 0, 0, 2, 2)
    assert lib.vdnn_maxpool_bwd_in_place_ok(g) == 1
    rng = np.random.default_rng(h + w)
    x = relu(rng.standard_normal((n, c, h, w)).astype(np.float32))
    dy = rng.standard_normal((n, c, h // 2, w // 2)).astype(np.float32)
    ctx = be.Context(pool_bytes=1 << 30)
    try:
        if bf16:
            check(lib.vdnn_ctx_set_activation_dtype(ctx.handle, 1))
            x, dy = oracle.round_bf16(x), oracle.round_bf16(dy)
        dt = np.uint16 if bf16 else np.float32
        enc = (lambda a: to_bf16_bits(a)) if bf16 else (lambda a: a)
        announce("pool backward over its input", n, c, h, w, "bf16" if bf16 else "f32")
        with Dev(ctx) as d:
            for entry in (lib.vdnn_maxpool_bwd, lib.vdnn_maxpool_bwd_relu):
                a, cdy, over, apart = d.up(enc(x), dt), d.up(enc(dy), dt), d.up(enc(x), dt), d.empty(x.shape, dt)
                check(entry(ctx.handle, None, g, a.ptr, None, cdy.ptr, apart.ptr))
                check(entry(ctx.handle, None, g, over.ptr, None, cdy.ptr, over.ptr))
                assert np.array_equal(over.download(x.shape, dt), apart.download(x.shape, dt))
    finally:
        ctx.close()


def test_pool_shapes_that_cannot_write_over_their_input_say_so():
    ctx = be.Context(pool_bytes=1 << 30)
    try:
        for geom in ((2, 4, 13, 13, 0, 3, 3, 0, 0, 2, 2), (2, 4, 14, 14, 0, 2, 2, 0, 0, 2, 2), (1, 2, 9, 12, 0, 2, 2, 0, 0, 2, 2)):
            g = be.shape(*geom)
            assert lib.vdnn_maxpool_bwd_in_place_ok(g) == 0
            n, c, h, w = geom[:4]
            x = relu(np.random.default_rng(1).standard_normal((n, c, h, w)).astype(np.float32))
            P, Q = lib.vdnn_out_dim(h, 0, g.r, g.stride_h), lib.vdnn_out_dim(w, 0, g.s, g.stride_w)
            announce("pool backward over its input refused", geom)
            with Dev(ctx) as d:
                over, cdy = d.up(x), d.up(np.ones((n, c, P, Q), np.float32))
                assert lib.vdnn_maxpool_bwd(ctx.handle, None, g, over.ptr, None, cdy.ptr, over.ptr) != 0
                assert np.array_equal(over.download(x.shape), x)
    finally:
        ctx.close()


@pytest.mark.parametrize("cnn,batch,algo,bf16", [(None, 4, VDNN_MEMORY_OPT_ALGO, False), (ALEXNET_LRN, 4, VDNN_MEMORY_OPT_ALGO, False),
                                                 (OVERFEAT, 3, VDNN_MEMORY_OPT_ALGO, False), (VGG16_128, 2, VDNN_PERF_OPT_ALGO, False),
                                                 (VGG16_128, 2, VDNN_MEMORY_OPT_ALGO, True)])
def test_networks_that_write_gradients_over_inputs_keep_every_bit(cnn, batch, algo, bf16):
    def make(policy, **kw):
        if cnn is None:
            return Network(layers=small_specs(batch), policy=policy, algo=algo, capture=True, seed=3, bf16=bf16, **kw)
        return Network(cnn, policy, algo, batch, capture=True, seed=3, bf16=bf16, **kw)

    announce("in-place networks", cnn, batch, "BASELINE")
    with make(BASELINE) as net:
        plain = run_steps(net, 2)
        specs = list(net.specs)
    assert all(np.isfinite(v) for v in plain["loss"])
    # separate ReLU layers: the gradient goes over the input where a convolution or pooling layer lies below
    for policy, kw in ((VDNN_NONE, {}), (VDNN_ALL, {}), (VDNN_CONV, {"offload_lag": 3})):
        announce("in-place networks", cnn, batch, "policy", policy, kw, "unfused rectifiers")
        with make(policy, refined=True, **kw) as net:
            peak_apart = net_peak(net)
        with make(policy, refined=True, in_place=True, **kw) as net:
            got = run_steps(net, 2)
            peak = net.stats()["peak_bytes_in_use"]
        assert_bit_identical(got, plain, "policy %d %s" % (policy, kw))
        assert peak <= peak_apart + (512 * 512 * 9 * 4 if algo == VDNN_PERF_OPT_ALGO else 0)   # (see below)
    # fused rectifiers: every convolution above the first and every 2x2 pooling layer
    shrinks = 0
    for policy, kw in ((VDNN_NONE, {}), (VDNN_CONV, {}), (VDNN_ALL, {}), (VDNN_ALL, {"host_sync": True}),
                       (VDNN_ALL, {"offload_lag": 6, "prefetch_depth": 3}), (VDNN_ALL, {"unfused_optimizer": True}),
                       (VDNN_ALL, {"compress": True}), (VDNN_ALL, {"compress": True, "keep_packed": True}),
                       (VDNN_CONV, {"compress": True, "prefetch_within_peak": True, "offload_lag": 4}),
                       # the first layer's output computed again before its consumer's backward instead of kept or moved
                       (VDNN_NONE, {"recompute_first": True}), (VDNN_ALL, {"recompute_first": True, "offload_lag": 2}),
                       (VDNN_ALL, {"recompute_first": True, "compress": True, "keep_packed": True}),
                       (VDNN_CONV, {"recompute_first": True, "compress": True, "host_sync": True}),
                       (VDNN_ALL, {"recompute_first": True, "unfused_optimizer": True, "prefetch_depth": 2}),
                       # a budget halfway between the floor and what the schedule holds unplaced; the plan chooses the lag
                       (VDNN_ALL, {"recompute_first": True, "compress": True, "plan_packed_fraction": 0.7, "hbm_budget_bytes": "middle",
                                   "offload_lag": -1, "prefetch_within_peak": True})):
        if kw.get("hbm_budget_bytes") == "middle":
            rest = {k: v for k, v in kw.items() if k != "hbm_budget_bytes"}
            with make(policy, refined=True, fuse=True, in_place=True, plan_only=True, hbm_budget_bytes=1, **rest) as probe:
                floor = probe.plan_peak_bytes()
            with make(policy, refined=True, fuse=True, in_place=True, plan_only=True, hbm_budget_bytes=1 << 50, **rest) as probe:
                ceiling = probe.plan_peak_bytes()
            kw = dict(kw, hbm_budget_bytes=(floor + ceiling) // 2)
        announce("in-place networks", cnn, batch, "policy", policy, kw, "fused rectifiers")
        with make(policy, refined=True, fuse=True, **{k: v for k, v in kw.items() if k not in ("recompute_first", "hbm_budget_bytes")}) as net:
            peak_apart = net_peak(net)
        with make(policy, refined=True, fuse=True, in_place=True, **kw) as net:
            got = run_steps(net, 2)
            peak = net.stats()["peak_bytes_in_use"]
            offloaded = {l for l in range(net.num_layers) if net.is_offloaded(l)}
            if kw.get("recompute_first"):   # (every table here starts convolution, ReLU, consumer)
                assert net.recomputed_layer() == 2 and not net.is_offloaded(0) and not net.is_offloaded(2)
        if kw.get("compress"):   # a layer whose input is a packed stream expands it itself and masks as in BASELINE
            offloaded = {l for l in offloaded if not rectified(specs, l)}
        assert_fused_matches(got, plain, specs, "policy %d %s" % (policy, kw), offloaded)
        if "hbm_budget_bytes" in kw:
            continue   # (a budget keeps on the device what fits: more than the policy's own offload set would)
        # The in-place order keeps a filter-sized gradient block while backward filter runs. In the perf-optimal mode that
        # pass holds its Winograd workspace at the same time, and at a batch of two the block (9.4 MB for 512 x 512 x 3 x 3)
        # outweighs the activation gradient it saves (3.2 MB): the peak may exceed the separate-blocks one by that block.
        slack = 512 * 512 * 9 * 4 if algo == VDNN_PERF_OPT_ALGO else 0
        assert peak <= peak_apart + slack
        shrinks += peak < peak_apart
    if cnn == VGG16_128:   # (the small tables' peaks are the parameters and the staging area)
        assert shrinks > 0, "writing gradients over inputs never lowered a peak"


def net_peak(net):
    for _ in range(2):
        assert net.forwardPropagation() == 0 and net.backwardPropagation() == 0
    net.synchronize()
    return net.stats()["peak_bytes_in_use"]


@pytest.mark.parametrize("cnn,batch,algo,bf16", [(VGG16_128, 2, VDNN_MEMORY_OPT_ALGO, False), (VGG16_128, 2, VDNN_MEMORY_OPT_ALGO, True),
                                                 (ALEXNET_LRN, 4, VDNN_PERF_OPT_ALGO, False), (OVERFEAT, 3, VDNN_MEMORY_OPT_ALGO, True)])
def test_schedule_options_drawn_at_random_keep_every_bit(cnn, batch, algo, bf16):
    """The options that change when and where a tensor lives (policy, lifetimes, lag, depth of prefetch, packing, keeping
    packed blocks, placement by a budget between the plan's floor and what fits unplaced, gradients over inputs, the
    first layer computed again, the update apart, host synchronisation) combined at random from a fixed seed: every
    combination must leave the losses, outputs and gradients of two steps as BASELINE leaves them."""
    import random
    rnd = random.Random(hash((cnn, batch, bf16)) & 0xFFFF)

    def make(policy, **kw):
        return Network(cnn, policy, algo, batch, capture=True, seed=3, bf16=bf16, **kw)

    announce("random schedules", cnn, batch, "bf16" if bf16 else "f32", "BASELINE")
    with make(BASELINE) as net:
        plain = run_steps(net, 2)
        specs = list(net.specs)
    for _ in range(10):
        policy = rnd.choice([VDNN_NONE, VDNN_CONV, VDNN_ALL])
        kw = dict(refined=True, fuse=True, in_place=rnd.random() < 0.6, recompute_first=rnd.random() < 0.5, host_sync=rnd.random() < 0.15,
                  offload_lag=rnd.choice([0, 0, 2, 6, 14, -1]), prefetch_depth=rnd.choice([1, 1, 2, 3]),
                  prefetch_within_peak=rnd.random() < 0.3, unfused_optimizer=rnd.random() < 0.2, compress=rnd.random() < 0.6)
        if kw["compress"]:
            kw["keep_packed"] = rnd.random() < 0.5
            if rnd.random() < 0.5:
                kw["plan_packed_fraction"] = 0.7
                with make(policy, plan_only=True, hbm_budget_bytes=1, **kw) as probe:
                    floor = probe.plan_peak_bytes()
                with make(policy, plan_only=True, hbm_budget_bytes=1 << 50, **kw) as probe:
                    ceiling = probe.plan_peak_bytes()
                kw["hbm_budget_bytes"] = int(floor + (ceiling - floor) * rnd.choice([0.0, 0.3, 0.6, 1.0]))
        announce("random schedules", cnn, batch, "bf16" if bf16 else "f32", "policy", policy, kw)
        with make(policy, **kw) as net:
            got = run_steps(net, 2)
            offloaded = {l for l in range(net.num_layers) if net.is_offloaded(l)}
        if kw["compress"]:
            offloaded = {l for l in offloaded if not rectified(specs, l)}
        assert_fused_matches(got, plain, specs, "policy %d %s" % (policy, kw), offloaded)
