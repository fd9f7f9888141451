"""A small training loop written against the layer / optimizer mirrors, as the reference's
examples write theirs (`examples/function_fitting.rs`, `examples/mnist_cnn/src/main.rs:262-311`:
zero_grad, forward, loss, backward with the parameters, optimizer step), and the same loop in
float64 numpy.  Model: Linear(3,16) -> tanh -> Linear(16,2), loss = sum((y - t)^2) / batch."""

import numpy as np


def run(fe, kind, optimizer: str, steps: int, seed: int = 5):
    """Trains on backend `kind`; returns (losses, final parameters as arrays)."""
    from harp_amd.frontend.tensor import _INPUT_BUFFER_CACHE
    from harp_amd.workloads import tanh_exact
    fe.set_device_str(kind)
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1, 1, (32, 3)).astype(np.float32)
    t = np.stack([np.sin(x.sum(1)), np.cos(x[:, 0])], 1).astype(np.float32)
    try:
        with fe.exact_mode():
            l1, l2 = fe.layers.Linear(3, 16), fe.layers.Linear(16, 2)
            params = l1.parameters() + l2.parameters()
            opt = {"sgd": lambda: fe.optim.SGD(params, 0.05),
                   "momentum": lambda: fe.optim.SGD(params, 0.05, momentum=0.9),
                   "adam": lambda: fe.optim.Adam(params, 0.01)}[optimizer]()
            xt, tt = fe.Tensor.input([32, 3]), fe.Tensor.input([32, 2])
            xt.set_data(x)
            tt.set_data(t)
            losses = []
            for _ in range(steps):
                opt.zero_grad()
                d = l2.forward(tanh_exact(l1.forward(xt))) - tt
                loss = (d * d).sum(1).sum(0).scale_exact(1.0 / 32)
                loss.backward_with_params([p.tensor() for p in params])
                opt.step(also=[loss])
                losses.append(float(loss.to_numpy()[0]))
            return losses, [p.to_numpy() for p in params]
    finally:
        _INPUT_BUFFER_CACHE.clear()


def run_numpy(fe, optimizer: str, steps: int, seed: int = 5):
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1, 1, (32, 3)).astype(np.float32).astype(np.float64)
    t = np.stack([np.sin(x.sum(1)), np.cos(x[:, 0])], 1).astype(np.float32).astype(np.float64)
    l1, l2 = fe.layers.Linear(3, 16), fe.layers.Linear(16, 2)
    p = [q.to_numpy().astype(np.float64) for q in l1.parameters() + l2.parameters()]
    vel = [np.zeros_like(q) for q in p]
    m = [np.zeros_like(q) for q in p]
    v = [np.zeros_like(q) for q in p]
    losses = []
    for step in range(1, steps + 1):
        w1, b1, w2, b2 = p
        h = np.tanh(x @ w1.T + b1)
        d = h @ w2.T + b2 - t
        losses.append(float((d * d).sum() / 32))
        dy = 2 * d / 32
        dh = dy @ w2 * (1 - h * h)
        g = [dh.T @ x, dh.sum(0), dy.T @ h, dy.sum(0)]
        for i in range(4):
            if optimizer == "sgd":
                p[i] = p[i] - 0.05 * g[i]
            elif optimizer == "momentum":
                vel[i] = 0.9 * vel[i] - 0.05 * g[i]
                p[i] = p[i] + vel[i]
            else:
                m[i] = 0.9 * m[i] + 0.1 * g[i]
                v[i] = 0.999 * v[i] + 0.001 * g[i] * g[i]
                p[i] = p[i] - 0.01 * (m[i] / (1 - 0.9 ** step)) / (np.sqrt(v[i] / (1 - 0.999 ** step)) + 1e-8)
    return losses, p
