"""float64 numpy statements of the two training steps, for checking what the backend computes
(the benchmark's result checks and the parity tests use them; they are plain mathematics, not the
reference's lowering).

`cnn_step`: the config-5 CNN (conv3x3 pad 1 + relu + maxpool2, twice; fc + relu; fc;
cross-entropy), forward and backward.  Max-pool ties share the gradient (every maximal element
receives it), as the graph's equality mask does.  `mlp_step`: the config-4 MLP with tanh and
mean-squared error."""

import numpy as np
def im2col(xp, kh, kw):
    n, c, H, W = xp.shape
    ho, wo = H - kh + 1, W - kw + 1
    cols = np.empty((n, ho, wo, c, kh, kw), xp.dtype)
    for i in range(kh):
        for j in range(kw):
            cols[:, :, :, :, i, j] = xp[:, :, i:i+ho, j:j+wo].transpose(0, 2, 3, 1)
    return cols.reshape(n, ho*wo, c*kh*kw), ho, wo
def conv_fwd(x, w, b):
    n = x.shape[0]; co, ci, kh, kw = w.shape
    xp = np.pad(x, ((0,0),(0,0),(1,1),(1,1)))
    cols, ho, wo = im2col(xp, kh, kw)
    y = cols @ w.reshape(co, -1).T
    return y.reshape(n, ho, wo, co).transpose(0, 3, 1, 2) + b[None, :, None, None], cols
def conv_bwd(g, x, w, cols):
    n, co, ho, wo = g.shape; _, ci, kh, kw = w.shape
    g2 = g.transpose(0, 2, 3, 1).reshape(n, ho*wo, co)
    dw = np.einsum('npo,npk->ok', g2, cols).reshape(w.shape)
    db = g.sum((0, 2, 3))
    dcols = (g2 @ w.reshape(co, -1)).reshape(n, ho, wo, ci, kh, kw)
    dxp = np.zeros((n, ci, ho+2, wo+2), g.dtype)
    for i in range(kh):
        for j in range(kw):
            dxp[:, :, i:i+ho, j:j+wo] += dcols[:, :, :, :, i, j].transpose(0, 3, 1, 2)
    return dxp[:, :, 1:-1, 1:-1], dw, db
def pool_fwd(x):
    n, c, h, w = x.shape
    xr = x.reshape(n, c, h//2, 2, w//2, 2).transpose(0, 1, 2, 4, 3, 5).reshape(n, c, h//2, w//2, 4)
    return xr.max(4), xr
def pool_bwd(g, xr, y):
    mask = (xr == y[..., None]).astype(g.dtype)
    gx = g[..., None] * mask
    n, c, ho, wo, _ = gx.shape
    return gx.reshape(n, c, ho, wo, 2, 2).transpose(0, 1, 2, 4, 3, 5).reshape(n, c, ho*2, wo*2)
def cnn_step(x, onehot, params):
    """float64 forward + backward; returns (loss, grads in the order of params)."""
    x = x.astype(np.float64); onehot = onehot.astype(np.float64)
    w1, b1, w2, b2, w3, b3, w4, b4 = [p.astype(np.float64) for p in params]
    z1, cols1 = conv_fwd(x, w1, b1); a1 = np.maximum(z1, 0); p1, xr1 = pool_fwd(a1)
    z2, cols2 = conv_fwd(p1, w2, b2); a2 = np.maximum(z2, 0); p2, xr2 = pool_fwd(a2)
    f = p2.reshape(x.shape[0], -1)
    z3 = f @ w3.T + b3; a3 = np.maximum(z3, 0)
    z4 = a3 @ w4.T + b4
    sh = z4 - z4.max(1, keepdims=True)
    lsm = sh - np.log(np.exp(sh).sum(1, keepdims=True))
    n = x.shape[0]
    loss = -(onehot * lsm).sum() / n
    gz4 = (np.exp(lsm) * onehot.sum(1, keepdims=True) - onehot) / n
    gw4 = gz4.T @ a3; gb4 = gz4.sum(0)
    gz3 = (gz4 @ w4) * (z3 >= 0)
    gw3 = gz3.T @ f; gb3 = gz3.sum(0)
    gp2 = (gz3 @ w3).reshape(p2.shape)
    gz2 = pool_bwd(gp2, xr2, p2) * (z2 >= 0)
    gp1, gw2, gb2 = conv_bwd(gz2, p1, w2, cols2)
    gz1 = pool_bwd(gp1, xr1, p1) * (z1 >= 0)
    _, gw1, gb1 = conv_bwd(gz1, x, w1, cols1)
    return loss, [gw1, gb1, gw2, gb2, gw3, gb3, gw4, gb4]


def mlp_step(arrays):
    """(loss, gradient of every parameter, network output) of the config-4 step for
    [x, target, w1, b1, w2, b2, ...], in float64."""
    x, t = arrays[0].astype(np.float64), arrays[1].astype(np.float64)
    ps = [p.astype(np.float64) for p in arrays[2:]]
    hs, pre = [x], []
    nl = len(ps) // 2
    for i in range(nl):
        z = hs[-1] @ ps[2 * i].T + ps[2 * i + 1]
        pre.append(z)
        hs.append(np.tanh(z) if i + 1 < nl else z)
    d = hs[-1] - t
    loss = (d * d).mean()
    gz = 2 * d / d.size
    grads = [None] * len(ps)
    for i in range(nl - 1, -1, -1):
        grads[2 * i] = gz.T @ hs[i]
        grads[2 * i + 1] = gz.sum(0)
        if i > 0:
            gz = (gz @ ps[2 * i]) * (1 - np.tanh(pre[i - 1]) ** 2)
    return loss, grads, hs[-1]
