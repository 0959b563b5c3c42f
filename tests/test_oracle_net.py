"""Pins the CPU checker's training step: a torch-autograd fixture of a small network with every layer
kind, the reference's layer tables, and a finite difference of the loss. No GPU."""
import numpy as np
import pytest

import oracle
from util import assert_close, golden

FC_GEMM, FC_CONV, RELU, SOFTMAX, POOL, LRN = 0, 2, 3, 6, 7, 10


def L(t, n, c, h, w, pad=0, stride=0, k=0, r=0):
    return oracle.LayerDesc(t, oracle.Shape(n, c, h, w, k, r, r, pad, pad, stride, stride), 0, 0, 0, 0)


def small_net_layers(n=4):
    return [L(FC_CONV, n, 3, 20, 20, 1, 1, 8, 3), L(RELU, n, 8, 20, 20), L(LRN, n, 8, 20, 20),
            L(POOL, n, 8, 20, 20, 0, 2, 0, 2), L(FC_CONV, n, 8, 10, 10, 2, 1, 12, 5), L(RELU, n, 12, 10, 10),
            L(POOL, n, 12, 10, 10, 0, 2, 0, 3), L(FC_GEMM, n, 192, 1, 1, 0, 0, 20, 1), L(RELU, n, 20, 1, 1),
            L(FC_GEMM, n, 20, 1, 1, 0, 0, 10, 1), L(SOFTMAX, n, 10, 1, 1)]


def load_small_net(f, net):
    net.input()[...] = f["x"]
    net.set_labels(f["labels"])
    for l in (0, 4, 7, 9):
        net.filter(l)[...] = f["w%d" % l].reshape(net.filter(l).shape)
        net.bias(l)[...] = f["b%d" % l]


@pytest.mark.parametrize("dbl", [False, True])
def test_small_net_step_against_torch_autograd(dbl):
    f = golden("small_net")
    oracle.set_accumulate_double(dbl)
    try:
        net = oracle.Net(layers=small_net_layers())
        load_small_net(f, net)
        ce = net.forward()
        assert abs(ce - float(f["ce"])) <= 1e-5 * abs(float(f["ce"]))
        for l in range(net.num_layers):
            assert_close(net.dst(l).reshape(f["dst%d" % l].shape), f["dst%d" % l], 1e-5, "dst %d" % l)
        w_before = {l: (net.filter(l).copy(), net.bias(l).copy()) for l in (0, 4, 7, 9)}
        net.backward()
        # grad[l] is d/d(src of l): the input gradient for l = 0, else the gradient of dst[l-1]
        assert_close(net.grad(0), f["dx"], 2e-5, "dx")
        for l in range(1, net.num_layers):
            want = f["ddst%d" % (l - 1)]
            assert_close(net.grad(l).reshape(want.shape), want, 2e-5, "grad %d" % l)
        # fused SGD: w_new = w + (-1e-5) * dW, no 1/N (layer.cu:593, 651-660)
        for l, (w0, b0) in w_before.items():
            dw = (net.filter(l).astype(np.float64) - w0) / -1e-5
            db = (net.bias(l).astype(np.float64) - b0) / -1e-5
            # the update is 1e-5 * gradient on top of O(0.1) weights: fp32 rounding of w bounds the check
            assert_close(dw.reshape(f["dw%d" % l].shape), f["dw%d" % l], 2e-2, "dw %d" % l)
            assert_close(db, f["db%d" % l], 2e-2, "db %d" % l)
    finally:
        oracle.set_accumulate_double(False)


def test_loss_decreases_along_the_step_direction():
    """A finite difference of 0.5*||y - label||^2 along the applied update confirms sign and scale."""
    f = golden("small_net")
    net = oracle.Net(layers=small_net_layers())
    load_small_net(f, net)
    target = net.label().reshape(4, 10).astype(np.float64)

    def sq_loss():
        net.forward()
        return 0.5 * np.sum((net.dst(10).reshape(4, 10).astype(np.float64) - target) ** 2)

    l0 = sq_loss()
    w0 = [net.filter(l).copy() for l in (0, 4, 7, 9)]
    b0 = [net.bias(l).copy() for l in (0, 4, 7, 9)]
    net.backward()
    gnorm2 = sum(np.sum(((net.filter(l).astype(np.float64) - w) / -1e-5) ** 2) for l, w in zip((0, 4, 7, 9), w0))
    gnorm2 += sum(np.sum(((net.bias(l).astype(np.float64) - b) / -1e-5) ** 2) for l, b in zip((0, 4, 7, 9), b0))
    # take a step 10x larger in the same direction: visible in fp32, still in the linear regime
    for l, w, b in zip((0, 4, 7, 9), w0, b0):
        net.filter(l)[...] = w + 10.0 * (net.filter(l) - w)
        net.bias(l)[...] = b + 10.0 * (net.bias(l) - b)
    l1 = sq_loss()
    predicted = -1e-4 * gnorm2
    assert l1 < l0
    assert abs((l1 - l0) - predicted) <= 0.1 * abs(predicted)


@pytest.mark.parametrize("cnn,layers,batch", [(0, 19, 128), (7, 21, 128), (1, 19, 128), (3, 37, 64), (4, 37, 128), (5, 37, 256)])
def test_tables_chain_like_the_reference(cnn, layers, batch):
    net = oracle.Net(cnn=cnn, batch=1)
    assert net.num_layers == layers
    for l in range(net.num_layers - 1):
        a, b = net.dst_shape(l), net.src_shape(l + 1)
        assert int(np.prod(a)) == int(np.prod(b))  # sanityCheck, network.cu:857-871
        if net.desc[l + 1].type != FC_GEMM:
            assert a == b
    assert net.dst_shape(net.num_layers - 1) == (1, 1000, 1, 1)
    net.close()
    full = oracle.lib.orc_net_create  # default batch of the table
    assert full is not None


def test_vgg16_flop_count_matches_the_table():
    net = oracle.Net(cnn=4, batch=1)
    flops = 0
    for d in net.desc:
        if d.type in (FC_CONV, FC_GEMM):
            flops += 2 * d.c_out * d.h_out * d.w_out * d.g.c * d.g.r * d.g.s
    assert abs(3 * flops / 1e9 - 92.82) < 0.01  # GFLOP per image and step
    net.close()


def test_alexnet_lrn_batch2_step_runs_and_is_finite():
    net = oracle.Net(cnn=7, batch=2)
    net.init_seeded(1)
    loss = net.forward()
    assert np.isfinite(loss) and 5.0 < loss < 9.0  # around ln(1000) = 6.9 for an untrained net
    y = net.dst(net.num_layers - 1).reshape(2, 1000)
    assert np.allclose(y.sum(axis=1), 1.0, atol=1e-5)
    net.backward()
    assert all(np.isfinite(net.grad(l)).all() for l in range(net.num_layers))
    assert np.abs(net.grad(0)).max() > 0
    net.close()


CONV, TANH, SIGMOID = 1, 4, 5


def drawn_table(rnd):
    """A layer table from a seeded generator: one to three convolutions (windows 1 to 5, strides, paddings) with ReLU /
    tanh / sigmoid, LRN and 2x2 or 3x3 pooling between them, one or two fully connected layers, softmax."""
    n = rnd.randint(1, 4)
    c, h, w = rnd.choice([1, 3, 4]), rnd.randint(10, 22), rnd.randint(10, 22)
    t = []
    for _ in range(rnd.randint(1, 3)):
        k, r = rnd.choice([4, 8, 12, 17]), rnd.choice([1, 3, 3, 5])
        pad, stride = rnd.choice([0, r // 2, r // 2]), rnd.choice([1, 1, 2])
        t.append(L(rnd.choice([CONV, FC_CONV]), n, c, h, w, pad, stride, k, r))
        h, w, c = (h + 2 * pad - r) // stride + 1, (w + 2 * pad - r) // stride + 1, k
        act = rnd.choice([RELU, RELU, TANH, SIGMOID, None])
        if act is not None:
            t.append(L(act, n, c, h, w))
        if rnd.random() < 0.3 and c >= 5:
            t.append(L(LRN, n, c, h, w))
        if rnd.random() < 0.6 and h >= 4 and w >= 4:
            win = rnd.choice([2, 2, 3])
            t.append(L(POOL, n, c, h, w, 0, 2, 0, win))
            h, w = (h - win) // 2 + 1, (w - win) // 2 + 1
        if h < 5 or w < 5:
            break
    feat = c * h * w
    for depth in range(rnd.randint(1, 2)):
        out = rnd.choice([7, 10, 16])
        t.append(L(FC_GEMM, n, feat, 1, 1, 0, 0, out, 1))
        feat = out
        if depth == 0 and rnd.random() < 0.5:
            t.append(L(rnd.choice([RELU, TANH]), n, feat, 1, 1))
    if t[-1].type != FC_GEMM:
        t.pop()
    t.append(L(SOFTMAX, n, feat, 1, 1))
    return t


@pytest.mark.parametrize("index", range(10))
def test_drawn_layer_tables_against_torch_autograd(index):
    """The checker's step on tables the fixture does not have, against torch built at test time in float64: every
    layer's output, the reported loss, every layer's input gradient (the reference's: no 1/N)."""
    import random
    import torch
    F = torch.nn.functional
    rnd = random.Random(500 + index)
    table = drawn_table(rnd)
    oracle.set_accumulate_double(True)
    try:
        net = oracle.Net(layers=table)
        net.init_seeded(index + 1)
        x = torch.tensor(net.input().astype(np.float64), requires_grad=True)
        labels = net.label().reshape(table[-1].g.n, -1)
        cur, outs, params = x, [], {}
        for l, d in enumerate(table):
            g = d.g
            if d.type in (CONV, FC_CONV):
                wt = torch.tensor(net.filter(l).astype(np.float64).reshape(g.k, g.c, g.r, g.s))
                bt = torch.tensor(net.bias(l).astype(np.float64))
                cur = F.conv2d(cur, wt, bt, stride=(g.stride_h, g.stride_w), padding=(g.pad_h, g.pad_w))
            elif d.type == FC_GEMM:
                wt = torch.tensor(net.filter(l).astype(np.float64).reshape(g.k, g.c))
                bt = torch.tensor(net.bias(l).astype(np.float64))
                cur = F.linear(cur.reshape(g.n, -1), wt, bt)
            elif d.type == RELU:
                cur = F.relu(cur)
            elif d.type == TANH:
                cur = torch.tanh(cur)
            elif d.type == SIGMOID:
                cur = torch.sigmoid(cur)
            elif d.type == LRN:
                cur = F.local_response_norm(cur, 5, alpha=1e-4, beta=0.75, k=2.0)
            elif d.type == POOL:
                cur = F.max_pool2d(cur, g.r, g.stride_h)
            elif d.type == SOFTMAX:
                cur = F.softmax(cur.reshape(g.n, -1), dim=1)
            cur.retain_grad()
            outs.append(cur)
        target = torch.tensor(labels.astype(np.float64))
        ce_sum = -(target * torch.log(outs[-1])).sum()
        ce = net.forward()
        for l in range(len(table)):
            assert_close(net.dst(l).reshape(tuple(outs[l].shape)), outs[l].detach().numpy(), 2e-5, "dst %d" % l)
        net.backward()
        # the reference starts backward from dy = y - label at the softmax OUTPUT and passes it through the softmax
        # layer's own backward (network.cu:1042-1054): the gradient of 0.5 * ||softmax(z) - label||^2, no 1/N
        (0.5 * ((outs[-1] - target) ** 2).sum()).backward()
        want_ce = float(ce_sum.detach()) / table[-1].g.n   # the reported loss: cross-entropy, mean over the batch
        assert abs(ce - want_ce) <= 1e-5 * abs(want_ce)
        assert_close(net.grad(0), x.grad.numpy(), 5e-5, "dx")
        for l in range(1, len(table) - 1):
            want = outs[l - 1].grad.numpy()
            assert_close(net.grad(l).reshape(want.shape), want, 5e-5, "grad %d" % l)
    finally:
        oracle.set_accumulate_double(False)
