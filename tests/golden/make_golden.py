"""Writes the golden fixtures under tests/golden/ with torch on the CPU (an independent library, not
the reference: the reference has no tests, fixtures or runnable build). Run once in the development
container:  python tests/golden/make_golden.py

Every expected value is computed in float64 and stored as float32 next to its float32 inputs.
"""
import os

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.abspath(__file__))
torch.manual_seed(20240917)
torch.set_num_threads(4)


def rnd(*shape, scale=1.0):
    return (torch.randn(*shape, dtype=torch.float64) * scale).float().double()


def save(name, **arrays):
    out = {}
    for k, v in arrays.items():
        if isinstance(v, torch.Tensor):
            v = v.detach().numpy()
        v = np.asarray(v)
        out[k] = v.astype(np.float32) if v.dtype == np.float64 else v
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **out)
    print("wrote", name, {k: tuple(v.shape) for k, v in out.items()})


# ---- convolution: every filter geometry the three networks use, at small extents -------------------
CONV_CASES = {
    # name: (n, c, h, w, k, r, s, pad, stride)
    "vgg_3x3_p1": (2, 5, 9, 11, 7, 3, 3, 1, 1),
    "alex_11x11_s4": (2, 3, 35, 39, 6, 11, 11, 0, 4),
    "alex_5x5_p2": (2, 4, 9, 9, 5, 5, 5, 2, 1),
    "overfeat_5x5_p0": (2, 4, 10, 12, 5, 5, 5, 0, 1),
    "overfeat_6x6_to_1x1": (3, 8, 6, 6, 10, 6, 6, 0, 1),
    "overfeat_1x1": (3, 12, 1, 1, 9, 1, 1, 0, 1),
    "odd_3x3_s2_p1": (2, 3, 10, 13, 4, 3, 3, 1, 2),
}
for name, (n, c, h, w, k, r, s, pad, stride) in CONV_CASES.items():
    x = rnd(n, c, h, w).requires_grad_()
    wt = rnd(k, c, r, s, scale=0.3).requires_grad_()
    b = rnd(k, scale=0.5).requires_grad_()
    y = F.conv2d(x, wt, b, stride=stride, padding=pad)
    dy = rnd(*y.shape)
    y.backward(dy)
    save("conv_" + name, geom=np.array([n, c, h, w, k, r, s, pad, pad, stride, stride], np.int32),
         x=x, w=wt, b=b, y=y, dy=dy, dx=x.grad, dw=wt.grad, db=b.grad)

# ---- fully connected ---------------------------------------------------------------------------------
x = rnd(6, 37).requires_grad_()
wt = rnd(29, 37, scale=0.2).requires_grad_()
b = rnd(29).requires_grad_()
y = F.linear(x, wt, b)
dy = rnd(*y.shape)
y.backward(dy)
save("fc", x=x, w=wt, b=b, y=y, dy=dy, dx=x.grad, dw=wt.grad, db=b.grad)

# ---- max pooling: continuous random data has no ties, so the tie rule does not enter ---------------
for name, (n, c, h, w, win, stride) in {"pool_3x3_s2": (2, 3, 13, 15, 3, 2), "pool_2x2_s2": (2, 3, 12, 10, 2, 2),
                                        "pool_2x2_s2_odd": (1, 2, 7, 9, 2, 2)}.items():
    x = rnd(n, c, h, w).requires_grad_()
    y = F.max_pool2d(x, win, stride)
    dy = rnd(*y.shape)
    y.backward(dy)
    save(name, geom=np.array([n, c, h, w, 0, win, win, 0, 0, stride, stride], np.int32), x=x, y=y, dy=dy, dx=x.grad)

# ---- ReLU --------------------------------------------------------------------------------------------
x = rnd(4, 3, 5, 7).requires_grad_()
y = F.relu(x)
dy = rnd(*y.shape)
y.backward(dy)
save("relu", x=x, y=y, dy=dy, dx=x.grad)

# ---- LRN (window 5, alpha 1e-4, beta 0.75, k 2) and a stronger alpha so the normaliser matters ------
for name, alpha, scale in (("lrn", 1e-4, 1.0), ("lrn_large_inputs", 1e-4, 60.0)):
    x = rnd(2, 9, 4, 5, scale=scale).requires_grad_()
    y = F.local_response_norm(x, 5, alpha=alpha, beta=0.75, k=2.0)
    dy = rnd(*y.shape)
    y.backward(dy)
    save(name, x=x, y=y, dy=dy, dx=x.grad)

# ---- softmax, softmax-CE -----------------------------------------------------------------------------
x = rnd(5, 17, scale=3.0).requires_grad_()
y = F.softmax(x, dim=1)
dy = rnd(*y.shape)
y.backward(dy)
save("softmax", x=x, y=y, dy=dy, dx=x.grad)

x = rnd(6, 11, scale=2.0).requires_grad_()
labels = torch.randint(0, 11, (6,))
loss = F.cross_entropy(x, labels)
loss.backward()
save("softmax_ce", x=x, labels=labels.numpy().astype(np.int32), prob=F.softmax(x, dim=1), loss=loss.reshape(1), dx=x.grad)

# ---- a small network with every layer kind, trained one step the way the reference does ------------
# dy_last = softmax(z) - label (network.cu:1042-1054) is the gradient of 0.5*||softmax(z) - label||^2.
N = 4
x0 = rnd(N, 3, 20, 20)
params = {
    "w0": rnd(8, 3, 3, 3, scale=0.27), "b0": rnd(8, scale=0.1),      # conv 3x3 p1
    "w4": rnd(12, 8, 5, 5, scale=0.1), "b4": rnd(12, scale=0.1),     # conv 5x5 p2
    "w7": rnd(20, 12 * 4 * 4, scale=0.1), "b7": rnd(20, scale=0.1),  # fc
    "w9": rnd(10, 20, scale=0.3), "b9": rnd(10, scale=0.1),          # fc
}
for p in params.values():
    p.requires_grad_()
labels = torch.randint(0, 10, (N,))
target = F.one_hot(labels, 10).double()
acts = []


def keep(t):
    t.retain_grad()
    acts.append(t)
    return t


x0.requires_grad_()
a = keep(F.conv2d(x0, params["w0"], params["b0"], padding=1))       # 0 conv   -> 8x20x20
a = keep(F.relu(a))                                                  # 1 relu
a = keep(F.local_response_norm(a, 5, alpha=1e-4, beta=0.75, k=2.0))  # 2 lrn
a = keep(F.max_pool2d(a, 2, 2))                                      # 3 pool 2x2 s2 -> 8x10x10
a = keep(F.conv2d(a, params["w4"], params["b4"], padding=2))        # 4 conv   -> 12x10x10
a = keep(F.relu(a))                                                  # 5 relu
a = keep(F.max_pool2d(a, 3, 2))                                      # 6 pool 3x3 s2 -> 12x4x4
a = keep(F.linear(a.reshape(N, -1), params["w7"], params["b7"]))     # 7 fc -> 20
a = keep(F.relu(a))                                                  # 8 relu
a = keep(F.linear(a, params["w9"], params["b9"]))                    # 9 fc -> 10
a = keep(F.softmax(a, dim=1))                                        # 10 softmax
loss = 0.5 * ((a - target) ** 2).sum()
loss.backward()
out = {"x": x0, "labels": labels.numpy().astype(np.int32), "dx": x0.grad,
       "ce": -(target * torch.log(a)).sum() / N}
for i, t in enumerate(acts):
    out["dst%d" % i] = t
    out["ddst%d" % i] = t.grad
for k, p in params.items():
    out[k] = p
    out["d" + k] = p.grad
save("small_net", **out)
