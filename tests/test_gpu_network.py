"""GPU parity of whole training steps through the Network C ABI.

 1. a small network with every layer kind against a torch-autograd fixture;
 2. every memory policy, with events or with the reference's per-layer host syncs, gives
    bit-identical loss, gradients and post-step filters to BASELINE;
 3. the reference's networks (reduced batch) against the CPU checker, layer by layer:
    outputs to 1e-4 relative (max norm); gradients to 1e-4 relative in the L2 norm with at most
    1e-4 of the elements off by more than 1e-3 of the tensor's maximum (a ReLU or max-pool
    decision that flips on a last-bit difference changes single elements by O(1));
 4. an offloaded and prefetched tensor is byte-identical (the network input after a step).
"""
import hashlib

import numpy as np
import pytest

import oracle
from gpu_util import announce
from test_oracle_net import load_small_net, small_net_layers
from util import assert_close, assert_close_bf16, golden, rel_err
from vdnn_implementation_amd import (ALEXNET, ALEXNET_LRN, BASELINE, OVERFEAT, VDNN_ALL, VDNN_CONV, VDNN_MEMORY_OPT_ALGO,
                                     VDNN_NONE, VDNN_PERF_OPT_ALGO, VGG16_128, enums)
from vdnn_implementation_amd.network import Network, layer_spec

pytestmark = pytest.mark.gpu
POLICIES = [BASELINE, VDNN_NONE, VDNN_CONV, VDNN_ALL]


def small_specs(n=4):
    return [layer_spec(enums.FC_CONV, n, 3, 20, 20, 1, 1, 8, 3), layer_spec(enums.RELU, n, 8, 20, 20),
            layer_spec(enums.LRN, n, 8, 20, 20), layer_spec(enums.POOL, n, 8, 20, 20, 0, 2, 0, 2),
            layer_spec(enums.FC_CONV, n, 8, 10, 10, 2, 1, 12, 5), layer_spec(enums.RELU, n, 12, 10, 10),
            layer_spec(enums.POOL, n, 12, 10, 10, 0, 2, 0, 3), layer_spec(enums.FC_GEMM, n, 192, 1, 1, 0, 0, 20, 1),
            layer_spec(enums.RELU, n, 20, 1, 1), layer_spec(enums.FC_GEMM, n, 20, 1, 1, 0, 0, 10, 1),
            layer_spec(enums.SOFTMAX, n, 10, 1, 1)]


@pytest.mark.parametrize("policy", POLICIES)
def test_small_net_against_torch_autograd(policy):
    f = golden("small_net")
    announce("small net golden, policy", policy)
    with Network(layers=small_specs(), policy=policy, capture=True) as net:
        net.set_input(f["x"])
        net.set_labels(f["labels"])
        for l in (0, 4, 7, 9):
            net.set_params(l, f["w%d" % l], f["b%d" % l])
        assert net.forwardPropagation() == 0
        assert abs(net.loss() - float(f["ce"])) <= 1e-4 * abs(float(f["ce"]))
        assert net.backwardPropagation() == 0
        for l in range(net.num_layers):
            assert_close(net.captured_dst(l).reshape(f["dst%d" % l].shape), f["dst%d" % l], 1e-4, "dst %d" % l)
        assert_close(net.captured_grad(0), f["dx"], 1e-4, "dx")
        for l in range(1, net.num_layers):
            want = f["ddst%d" % (l - 1)]
            assert_close(net.captured_grad(l).reshape(want.shape), want, 1e-4, "grad %d" % l)
        for l in (0, 4, 7, 9):
            w, b = net.get_params(l)
            dw = (w.astype(np.float64).reshape(f["w%d" % l].shape) - f["w%d" % l]) / -1e-5
            assert_close(dw, f["dw%d" % l], 2e-2, "dw %d" % l)  # bounded by fp32 rounding of w + 1e-5*dw


def run_steps(net, steps):
    out = {"loss": [], "grads": [], "dsts": []}
    for _ in range(steps):
        assert net.forwardPropagation() == 0
        out["loss"].append(np.float32(net.loss()))
        assert net.backwardPropagation() == 0
        out["grads"].append([net.captured_grad(l) for l in range(net.num_layers)])
        out["dsts"].append([net.captured_dst(l) for l in range(net.num_layers)])
    out["params"] = [net.get_params(l) for l in range(net.num_layers) if net.has_params(l)]
    out["input"] = net.get_input()
    return out


def assert_bit_identical(a, b, what):
    assert [x.tobytes() for x in a["loss"]] == [x.tobytes() for x in b["loss"]], what + ": loss"
    for s, (ga, gb) in enumerate(zip(a["grads"], b["grads"])):
        for l, (x, y) in enumerate(zip(ga, gb)):
            assert np.array_equal(x.view(np.uint32), y.view(np.uint32)), "%s: step %d gradient of layer %d" % (what, s, l)
    for s, (da, db) in enumerate(zip(a["dsts"], b["dsts"])):
        for l, (x, y) in enumerate(zip(da, db)):
            assert np.array_equal(x.view(np.uint32), y.view(np.uint32)), "%s: step %d output of layer %d" % (what, s, l)
    for i, ((wa, ba), (wb, bb)) in enumerate(zip(a["params"], b["params"])):
        assert np.array_equal(wa.view(np.uint32), wb.view(np.uint32)) and np.array_equal(ba.view(np.uint32), bb.view(np.uint32)), "%s: params %d" % (what, i)
    assert np.array_equal(a["input"].view(np.uint32), b["input"].view(np.uint32)), what + ": input after the step"


@pytest.mark.parametrize("cnn,batch,algo,bf16", [(None, 4, VDNN_MEMORY_OPT_ALGO, False), (ALEXNET_LRN, 4, VDNN_MEMORY_OPT_ALGO, False),
                                                 (OVERFEAT, 3, VDNN_MEMORY_OPT_ALGO, False), (VGG16_128, 2, VDNN_PERF_OPT_ALGO, False),
                                                 (None, 4, VDNN_MEMORY_OPT_ALGO, True), (VGG16_128, 2, VDNN_MEMORY_OPT_ALGO, True)])
def test_policies_are_bit_identical_to_baseline(cnn, batch, algo, bf16):
    def make(policy, host_sync=False, refined=False, **kw):
        if cnn is None:
            return Network(layers=small_specs(batch), policy=policy, algo=algo, capture=True, seed=3, host_sync=host_sync, refined=refined, bf16=bf16, **kw)
        return Network(cnn, policy, algo, batch, capture=True, seed=3, host_sync=host_sync, refined=refined, bf16=bf16, **kw)

    announce("policies bit-identical", cnn, batch, "BASELINE")
    with make(BASELINE) as net:
        base = run_steps(net, 2)
        x0 = None
    assert all(np.isfinite(v) for v in base["loss"])
    for policy in (VDNN_NONE, VDNN_CONV, VDNN_ALL):
        for host_sync in (False, True):
            announce("policies bit-identical", cnn, batch, "policy", policy, "host_sync", host_sync)
            with make(policy, host_sync) as net:
                got = run_steps(net, 2)
            assert_bit_identical(got, base, "policy %d host_sync %s" % (policy, host_sync))
        # the lifetime refinements (dead ReLU inputs released, early release of unread outputs,
        # in-place ReLU backward) change no value either
        announce("policies bit-identical", cnn, batch, "policy", policy, "refined lifetimes")
        with make(policy, refined=True) as net:
            got = run_steps(net, 2)
        assert_bit_identical(got, base, "policy %d refined" % policy)
        # scheduling slack (blocks recycled some layers after their offload, several tensors fetched ahead)
        # changes when things are copied, never what is computed
        for refined, lag, depth in ((False, 3, 2), (True, 6, 3), (False, 40, 1)):
            announce("policies bit-identical", cnn, batch, "policy", policy, "lag", lag, "depth", depth, "refined", refined)
            with make(policy, refined=refined, offload_lag=lag, prefetch_depth=depth) as net:
                got = run_steps(net, 2)
            assert_bit_identical(got, base, "policy %d lag %d depth %d" % (policy, lag, depth))


@pytest.mark.parametrize("variant", [0, 1], ids=["split-bf16", "winograd"])
def test_perf_optimal_steps_track_the_memory_optimal_ones(variant):
    """VGG16, two training steps in the perf-optimal mode (either variant) against the memory-optimal mode from the same
    seed (other kernels, other sums - not the same bits). Forward is continuous in its sums: every layer's output agrees
    within the mode's bound, 1e-4 of the tensor's largest element, and the loss within 1e-4 of its value. Backward is not
    - a rectifier's gate or a pooling window's winner can differ where two sums differ in their last bits, and one such
    element of a sparse gradient spreads over the layers below (measured: one element of 401408 at relu5_3, 7 % of
    conv1_2's) - so the gradients are held to 5e-2 of their norm (measured 8e-3) and the parameters after the steps to
    1e-4 (filters) / 2e-2 (biases, which start at zero and are their gradients) of their largest element. The kernels'
    own parity is what tests/test_gpu_kernels.py checks against the double-precision checker."""
    from vdnn_implementation_amd.backend import lib
    with Network(VGG16_128, BASELINE, VDNN_MEMORY_OPT_ALGO, 4, capture=True, seed=5) as net:
        want = run_steps(net, 2)
    before = lib.vdnn_conv_perf_variant(variant)
    try:
        announce("perf-optimal against memory-optimal", "variant", variant)
        with Network(VGG16_128, BASELINE, VDNN_PERF_OPT_ALGO, 4, capture=True, seed=5) as net:
            got = run_steps(net, 2)
    finally:
        lib.vdnn_conv_perf_variant(before)

    def close(x, y, what, tol=1e-4):
        scale = float(np.max(np.abs(y))) or 1.0
        err = float(np.max(np.abs(x.astype(np.float64) - y))) / scale
        assert err <= tol, "%s: %.3e of the largest element" % (what, err)

    for s in range(2):
        assert abs(float(got["loss"][s]) - float(want["loss"][s])) <= 1e-4 * abs(float(want["loss"][s])), "loss of step %d" % s
        for l, (x, y) in enumerate(zip(got["dsts"][s], want["dsts"][s])):
            close(x, y, "step %d output of layer %d" % (s, l))
        for l, (x, y) in enumerate(zip(got["grads"][s], want["grads"][s])):
            d = x.astype(np.float64) - y
            norm = float(np.sqrt((y.astype(np.float64) ** 2).sum())) or 1.0
            assert float(np.sqrt((d * d).sum())) <= 5e-2 * norm, "step %d gradient of layer %d" % (s, l)
    for i, ((wa, ba), (wb, bb)) in enumerate(zip(got["params"], want["params"])):
        close(wa, wb, "filter %d" % i)
        close(ba, bb, "bias %d" % i, 2e-2)
    assert any(not np.array_equal(x, y) for x, y in zip(got["dsts"][0], want["dsts"][0]))   # (the variant ran)


def layer_forward_on_checker(spec, src, w, b, bf16=False):
    """The checker's math for one layer on the given input (identical inputs, layer by layer). With bfloat16
    activations the products of forward and backward data take the filter rounded to bfloat16."""
    if bf16 and w is not None:
        w = oracle.round_bf16(w)
    g = oracle.shape(spec.n, spec.c, spec.h, spec.w, spec.k, spec.r, spec.s, spec.pad_h, spec.pad_w, spec.stride_h, spec.stride_w)
    t = spec.type
    if t in (enums.FC_CONV, enums.CONV):
        return oracle.conv_fwd(g, src, w, b)
    if t == enums.FC_GEMM:
        return oracle.fc_fwd(src.reshape(spec.n, -1), w.reshape(spec.k, -1), b).reshape(spec.n, spec.k, 1, 1)
    if t == enums.RELU:
        return oracle.relu_fwd(src)
    if t == enums.TANH:
        return oracle.tanh_fwd(src)
    if t == enums.SIGMOID:
        return oracle.sigmoid_fwd(src)
    if t == enums.LRN:
        return oracle.lrn_fwd(src)
    if t == enums.POOL:
        return oracle.maxpool_fwd(g, src)
    if t == enums.SOFTMAX:
        return oracle.softmax_fwd(src.reshape(spec.n, -1)).reshape(src.shape)
    raise AssertionError(t)


def layer_backward_on_checker(spec, src, dst, dy, w, b, bf16=False):
    """(dx, w_after, b_after) of one layer from the checker, lr = 1e-5 fused as in layer.cu:593."""
    wp = oracle.round_bf16(w) if bf16 and w is not None else w  # the filter as backward data multiplies it
    g = oracle.shape(spec.n, spec.c, spec.h, spec.w, spec.k, spec.r, spec.s, spec.pad_h, spec.pad_w, spec.stride_h, spec.stride_w)
    t = spec.type
    alpha = np.float32(1e-5 * -1.0)
    if t in (enums.FC_CONV, enums.CONV):
        return oracle.conv_bwd_data(g, dy, wp), oracle.conv_bwd_filter_sgd(g, src, dy, w, alpha), oracle.conv_bwd_bias_sgd(g, dy, b, alpha)
    if t == enums.FC_GEMM:
        x2, dy2, w2 = src.reshape(spec.n, -1), dy.reshape(spec.n, -1), w.reshape(spec.k, -1)
        return (oracle.fc_bwd_data(dy2, wp.reshape(spec.k, -1)).reshape(src.shape), oracle.fc_bwd_weight_sgd(x2, dy2, w2, alpha).reshape(w.shape),
                oracle.fc_bwd_bias_sgd(dy2, b, alpha))
    if t == enums.RELU:
        return oracle.relu_bwd(src, dst, dy), None, None
    if t == enums.TANH:
        return oracle.tanh_bwd(dst, dy), None, None
    if t == enums.SIGMOID:
        return oracle.sigmoid_bwd(dst, dy), None, None
    if t == enums.LRN:
        return oracle.lrn_bwd(src, dst, dy), None, None
    if t == enums.POOL:
        return oracle.maxpool_bwd(g, src, dst, dy), None, None
    if t == enums.SOFTMAX:
        return oracle.softmax_bwd(dst.reshape(spec.n, -1), dy.reshape(spec.n, -1)).reshape(src.shape), None, None
    raise AssertionError(t)


@pytest.mark.parametrize("cnn,batch,policy,algo", [
    (ALEXNET_LRN, 2, BASELINE, VDNN_MEMORY_OPT_ALGO),   # the CPU-runnable configuration, reduced batch
    (ALEXNET, 2, VDNN_ALL, VDNN_MEMORY_OPT_ALGO),
    (OVERFEAT, 2, VDNN_CONV, VDNN_MEMORY_OPT_ALGO),
    (VGG16_128, 1, VDNN_ALL, VDNN_PERF_OPT_ALGO),
])
def test_reference_networks_against_the_checker(cnn, batch, policy, algo):
    check_network_against_the_checker(cnn, batch, policy, algo)


@pytest.mark.parametrize("cnn,batch,policy,algo", [
    (ALEXNET_LRN, 2, VDNN_ALL, VDNN_MEMORY_OPT_ALGO),
    (VGG16_128, 1, VDNN_ALL, VDNN_PERF_OPT_ALGO),
    (OVERFEAT, 2, BASELINE, VDNN_MEMORY_OPT_ALGO),
])
def test_reference_networks_bf16_against_the_checker(cnn, batch, policy, algo):
    """bfloat16 activation storage: every layer within one bfloat16 unit in the last place of the checker's
    double-precision result on identical (bfloat16) inputs; ReLU and max-pool forward bit-exact."""
    check_network_against_the_checker(cnn, batch, policy, algo, bf16=True)


def smooth_specs(n=3):
    """A table with the two activation modes none of the reference's networks uses (layer.cu:362-369)."""
    return [layer_spec(enums.FC_CONV, n, 3, 16, 16, 1, 1, 8, 3), layer_spec(enums.TANH, n, 8, 16, 16),
            layer_spec(enums.POOL, n, 8, 16, 16, 0, 2, 0, 2), layer_spec(enums.FC_CONV, n, 8, 8, 8, 1, 1, 16, 3),
            layer_spec(enums.SIGMOID, n, 16, 8, 8), layer_spec(enums.FC_GEMM, n, 1024, 1, 1, 0, 0, 24, 1),
            layer_spec(enums.TANH, n, 24, 1, 1), layer_spec(enums.FC_GEMM, n, 24, 1, 1, 0, 0, 10, 1),
            layer_spec(enums.SOFTMAX, n, 10, 1, 1)]


@pytest.mark.parametrize("policy,refined", [(BASELINE, False), (VDNN_ALL, False), (VDNN_ALL, True)])
def test_tanh_and_sigmoid_layers_against_the_checker(policy, refined):
    check_network_against_the_checker(None, 3, policy, VDNN_MEMORY_OPT_ALGO, layers=smooth_specs(3), refined=refined)


def check_network_against_the_checker(cnn, batch, policy, algo, layers=None, refined=False, bf16=False):
    """Layer by layer on identical inputs: each layer's output and gradients, computed by the checker
    from the tensors the GPU run fed that layer, within 1e-4 relative (max norm); exact for ReLU and
    max-pool. End to end (where a ReLU or pooling decision that flips on a last-bit difference moves
    single elements by O(1)) the loss must agree to 1e-4 and the input gradient to 2e-2 in L2."""
    seed = 11
    o = oracle.Net(cnn=cnn, batch=batch) if layers is None else oracle.Net(layers=[
        oracle.LayerDesc(s.type, oracle.Shape(s.n, s.c, s.h, s.w, s.k, s.r, s.s, s.pad_h, s.pad_w, s.stride_h, s.stride_w), 0, 0, 0, 0)
        for s in layers])
    o.init_seeded(seed)
    o.set_bf16(bf16)
    oracle.set_accumulate_double(True)
    try:
        announce("network vs checker", cnn, batch, policy, algo)
        with (Network(cnn, policy, algo, batch, capture=True, seed=seed, bf16=bf16) if layers is None else
              Network(layers=layers, policy=policy, algo=algo, capture=True, seed=seed, refined=refined, bf16=bf16)) as net:
            # the product's own seeded draw equals the checker's, bit for bit (rounded to bfloat16 at upload)
            x0 = net.get_input()
            assert np.array_equal(x0.view(np.uint32), (oracle.round_bf16(o.input()) if bf16 else o.input()).view(np.uint32))
            before = {}
            for l in range(net.num_layers):
                if net.has_params(l):
                    w, b = net.get_params(l)
                    assert np.array_equal(w.view(np.uint32), o.filter(l).view(np.uint32)) and np.array_equal(b, o.bias(l))
                    before[l] = (w, b)
            want_loss = o.forward()
            assert net.forwardPropagation() == 0
            assert abs(net.loss() - want_loss) <= (3e-2 if bf16 else 1e-4) * abs(want_loss)
            o.backward()
            assert net.backwardPropagation() == 0
            L = net.num_layers
            dst = [net.captured_dst(l) for l in range(L)]
            grad = [net.captured_grad(l) for l in range(L)]
            target = o.label().reshape(dst[-1].shape)
            for l in range(L):
                spec = net.specs[l]
                src = (x0 if l == 0 else dst[l - 1]).reshape(net.src_shape(l))
                w, b = before.get(l, (None, None))
                want = layer_forward_on_checker(spec, src, w, b, bf16)
                exact = spec.type in (enums.RELU, enums.POOL)
                if exact:
                    assert np.array_equal(dst[l], want), "output of layer %d" % l
                elif bf16:
                    assert_close_bf16(dst[l], want, "output of layer %d" % l)
                else:
                    assert_close(dst[l], want, 1e-4, "output of layer %d" % l)
                dy = (dst[-1] - target) if l == L - 1 else grad[l + 1].reshape(net.dst_shape(l))
                if bf16 and l == L - 1:
                    dy = oracle.round_bf16(dy)
                want_dx, want_w, want_b = layer_backward_on_checker(spec, src, dst[l], dy, w, b, bf16)
                if exact and not (bf16 and spec.type == enums.POOL):
                    assert np.array_equal(grad[l], want_dx), "gradient of layer %d" % l
                elif bf16:
                    assert_close_bf16(grad[l], want_dx, "gradient of layer %d" % l)
                else:
                    assert_close(grad[l], want_dx, 1e-4, "gradient of layer %d" % l)
                if want_w is not None:
                    w1, b1 = net.get_params(l)
                    assert_close(w1, want_w, 1e-6, "filter of layer %d after the step" % l)
                    assert_close(b1, want_b, 1e-6, "bias of layer %d after the step" % l)
                    dw_got = (w1.astype(np.float64) - w) / -1e-5
                    dw_want = (want_w.astype(np.float64) - w) / -1e-5
                    if np.max(np.abs(dw_want)) > 1.0:  # otherwise below the fp32 resolution of w
                        l2 = np.linalg.norm(dw_got - dw_want) / np.linalg.norm(dw_want)
                        assert l2 <= 5e-2, "dW of layer %d: %.3e" % (l, l2)
            # end to end against the checker's own run
            assert_close(dst[-1], o.dst(L - 1), 5e-2 if bf16 else 1e-4, "network output")
            g0, w0 = grad[0].astype(np.float64).ravel(), o.grad(0).astype(np.float64).ravel()
            # bfloat16: one unit in the last place is 0.4-0.8 %, so ReLU / pooling decisions flip far more often
            # through 37 layers; the end-to-end gradient is only required to point the same way
            assert np.linalg.norm(g0 - w0) <= (0.5 if bf16 else 2e-2) * np.linalg.norm(w0), "input gradient, end to end"
            # offloaded then prefetched: the input block went to the host and back
            assert np.array_equal(net.get_input().view(np.uint32), x0.view(np.uint32))
            st = net.stats()
            if policy in (VDNN_ALL, VDNN_CONV):
                assert st["offload_bytes"] == st["prefetch_bytes"] > 0
    finally:
        oracle.set_accumulate_double(False)
        o.close()


def test_offload_moves_the_bytes_the_schedule_says():
    announce("offload byte counts, VGG16 batch 2")
    with Network(VGG16_128, VDNN_ALL, VDNN_MEMORY_OPT_ALGO, 2, seed=5) as net:
        x0 = net.get_input()
        assert net.forwardPropagation() == 0 and net.backwardPropagation() == 0
        st = net.stats()
        want = sum(int(np.prod(net.src_shape(l))) * 4 for l in range(net.num_layers - 1))
        assert st["offload_bytes"] == st["prefetch_bytes"] == want == st["pinned_bytes"]
        assert np.array_equal(net.get_input().view(np.uint32), x0.view(np.uint32))
        assert net.prefetch_trace() == [(l, l - 1) for l in range(36, 0, -1)]


def test_out_of_memory_under_a_cap_returns_minus_one_on_the_device():
    announce("cap: VDNN_NONE cannot fit, VDNN_ALL can")
    with Network(VGG16_128, VDNN_ALL, VDNN_MEMORY_OPT_ALGO, 4, seed=5) as net:
        assert net.forwardPropagation() == 0 and net.backwardPropagation() == 0
        need = net.stats()["peak_bytes_in_use"]
        loss_all = net.loss()
    cap = int(need * 1.03)
    with Network(VGG16_128, VDNN_ALL, VDNN_MEMORY_OPT_ALGO, 4, seed=5, cap_bytes=cap) as net:
        assert net.forwardPropagation(True) == 0 and net.backwardPropagation(True) == 0
        assert np.float32(net.loss()).tobytes() == np.float32(loss_all).tobytes()
    with Network(VGG16_128, VDNN_NONE, VDNN_MEMORY_OPT_ALGO, 4, seed=5, cap_bytes=cap) as net:
        assert net.forwardPropagation(True) == -1


def _losses_and_stats(cnn, policy, algo, batch, steps=2, **kw):
    with Network(cnn, policy, algo, batch, seed=11, **kw) as net:
        losses = []
        for _ in range(steps):
            assert net.forwardPropagation() == 0
            losses.append(np.float32(net.loss()).tobytes())
            assert net.backwardPropagation() == 0
        # one digest per layer with parameters, over the bytes of the filter and the bias after the last step
        for l in range(net.num_layers):
            if net.has_params(l):
                w, b = net.get_params(l)
                losses.append(hashlib.sha1(w.tobytes() + b.tobytes()).digest())
        return losses, net.stats()


@pytest.mark.parametrize("cnn,batch,algo,policies", [
    (OVERFEAT, 128, VDNN_MEMORY_OPT_ALGO, [VDNN_CONV]),                     # OverFeat-fast, batch 128, VDNN_CONV
    (VGG16_128, 64, VDNN_PERF_OPT_ALGO, [VDNN_ALL]),                        # VGG16, batch 64, VDNN_ALL, workspace kernels
    (VGG16_128, 128, VDNN_MEMORY_OPT_ALGO, [VDNN_NONE, VDNN_CONV, VDNN_ALL]),  # the four-policy comparison
], ids=["overfeat128_conv", "vgg16_64_all_perfopt", "vgg16_128_all_policies"])
def test_full_size_configurations_keep_the_baseline_losses(cnn, batch, algo, policies):
    """At full size no CPU result is affordable; what must hold at any size: every policy computes the
    bits BASELINE computes (the losses of two steps and a digest of every layer's parameters after them),
    moves the bytes its offload table says, and holds less device memory."""
    announce("full size", cnn, batch, algo, "BASELINE")
    base_losses, base_stats = _losses_and_stats(cnn, BASELINE, algo, batch)
    assert all(np.isfinite(np.frombuffer(b, np.float32)[0]) for b in base_losses[:2])
    for policy in policies:
        for refined in (False, True):
            announce("full size", cnn, batch, algo, "policy", policy, "refined", refined)
            losses, st = _losses_and_stats(cnn, policy, algo, batch, refined=refined)
            assert losses == base_losses
            assert st["offload_bytes"] == st["prefetch_bytes"]
            if policy != VDNN_NONE:
                assert st["offload_bytes"] > 0
                assert st["peak_bytes_in_use"] < base_stats["peak_bytes_in_use"]


def test_unfused_optimizer_gives_the_bits_of_the_fused_step():
    """dW / db kept in buffers and applied after backward: same losses and parameters as the fused
    update over three steps; with the step deferred, backward leaves the parameters alone."""
    announce("unfused optimizer, small net + AlexNet batch 4")
    for make in (lambda **kw: Network(layers=small_specs(4), policy=VDNN_ALL, algo=VDNN_MEMORY_OPT_ALGO, seed=3, **kw),
                 lambda **kw: Network(ALEXNET, VDNN_CONV, VDNN_PERF_OPT_ALGO, 4, seed=3, **kw)):
        with make() as fused:
            want_losses = fused.train(3)
            want = [fused.get_params(l) for l in range(fused.num_layers) if fused.has_params(l)]
        with make(unfused_optimizer=True) as net:
            got_losses = net.train(3)
            got = [net.get_params(l) for l in range(net.num_layers) if net.has_params(l)]
        assert got_losses.tobytes() == want_losses.tobytes() and len(got_losses) == 3
        for (wa, ba), (wb, bb) in zip(got, want):
            assert np.array_equal(wa.view(np.uint32), wb.view(np.uint32)) and np.array_equal(ba.view(np.uint32), bb.view(np.uint32))
        with make(unfused_optimizer=True, defer_optimizer=True) as net:
            layers = [l for l in range(net.num_layers) if net.has_params(l)]
            before = [net.get_params(l) for l in layers]
            assert net.forwardPropagation() == 0 and net.backwardPropagation() == 0
            for l, (w0, b0) in zip(layers, before):
                w1, b1 = net.get_params(l)
                assert np.array_equal(w0, w1) and np.array_equal(b0, b1)
            grads = [net.get_gradients(l) for l in layers]
            assert net.applyGradients() == 0
            lr = np.float32(-1e-5)
            for l, (w0, b0), (dw, db) in zip(layers, before, grads):
                w1, b1 = net.get_params(l)
                assert np.abs(dw).max() > 0
                # one fused multiply-add per element: within one rounding of the two-step float32 result
                assert_close(w1, w0.astype(np.float64) + np.float64(lr) * dw, 1e-6, "w += alpha dW")
                assert_close(b1, b0.astype(np.float64) + np.float64(lr) * db, 1e-6, "b += alpha db")
            # after the deferred step the parameters are those of one fused step
            with make() as fused:
                fused.train(1)
                for l in layers:
                    wf, bf = fused.get_params(l)
                    w1, b1 = net.get_params(l)
                    assert np.array_equal(wf.view(np.uint32), w1.view(np.uint32)) and np.array_equal(bf.view(np.uint32), b1.view(np.uint32))


def drawn_stack(rnd):
    """A layer table drawn from a seeded generator: one to four convolutions (windows 1 to 5, strides, paddings) with
    ReLU / tanh / sigmoid, LRN and 2x2 or 3x3 pooling between them, one to three fully connected layers, softmax."""
    n = rnd.randint(1, 5)
    c, h, w = rnd.choice([1, 3, 3, 4]), rnd.randint(12, 34), rnd.randint(12, 34)
    specs = []
    for _ in range(rnd.randint(1, 4)):
        k, r = rnd.choice([4, 8, 12, 16, 32, 64, 70]), rnd.choice([1, 3, 3, 3, 5])
        pad, stride = rnd.choice([0, r // 2, r // 2]), rnd.choice([1, 1, 1, 2])
        if h + 2 * pad < r or w + 2 * pad < r:
            break
        specs.append(layer_spec(rnd.choice([enums.CONV, enums.FC_CONV]), n, c, h, w, pad, stride, k, r))
        h, w, c = (h + 2 * pad - r) // stride + 1, (w + 2 * pad - r) // stride + 1, k
        act = rnd.choice([enums.RELU, enums.RELU, enums.RELU, enums.TANH, enums.SIGMOID, None])
        if act is not None:
            specs.append(layer_spec(act, n, c, h, w))
        if rnd.random() < 0.25 and c >= 5:
            specs.append(layer_spec(enums.LRN, n, c, h, w))
        if rnd.random() < 0.6 and h >= 4 and w >= 4:
            win, st = rnd.choice([(2, 2), (2, 2), (3, 2)])
            specs.append(layer_spec(enums.POOL, n, c, h, w, 0, st, 0, win))
            h, w = (h - win) // st + 1, (w - win) // st + 1
        if h < 3 or w < 3:
            break
    feat = c * h * w
    for depth in range(rnd.randint(1, 3)):
        out = rnd.choice([10, 16, 33, 64, 100])
        specs.append(layer_spec(enums.FC_GEMM, n, feat, 1, 1, 0, 0, out, 1))
        feat = out
        if depth < 2 and rnd.random() < 0.7:
            specs.append(layer_spec(enums.RELU, n, feat, 1, 1))
    if specs[-1].type == enums.RELU:
        specs.pop()
    specs.append(layer_spec(enums.SOFTMAX, n, feat, 1, 1))
    return specs


@pytest.mark.parametrize("index", range(12))
def test_drawn_layer_tables_against_the_checker(index):
    """Tables the built-in networks do not have (strided and unpadded convolutions in the middle, tanh and sigmoid,
    LRN behind any layer, odd planes), each under a policy, an algorithm mode, lifetimes and an element type drawn
    with it: layer by layer against the checker."""
    import random
    rnd = random.Random(1000 + index)
    specs = drawn_stack(rnd)
    policy = rnd.choice([enums.BASELINE, enums.VDNN_NONE, enums.VDNN_CONV, enums.VDNN_ALL])
    algo = rnd.choice([enums.VDNN_MEMORY_OPT_ALGO, enums.VDNN_PERF_OPT_ALGO])
    refined, bf16 = rnd.random() < 0.5, rnd.random() < 0.4
    check_network_against_the_checker(None, specs[0].n, policy, algo, layers=specs, refined=refined, bf16=bf16)
