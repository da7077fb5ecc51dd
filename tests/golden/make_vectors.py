"""Writes tests/golden/vectors.npz: small known-answer vectors for the path's functions, computed WITHOUT the oracle
and without the library, by numpy slicing / padding and by torch's CPU convolution and autograd in float64.
The reference holds no vectors of its own for this path; these pin the oracle (tests/test_golden_vectors.py, CPU) and
the HIP path (same file, GPU) to committed data from an independent implementation.

    python tests/golden/make_vectors.py        (numpy + torch on the CPU; rewrites vectors.npz deterministically)
"""
import os

import numpy as np
import torch


def main():
    rng = np.random.default_rng(0x5EED)
    out = {}
    # ---- pack / exchange / reduce / unpack: K row tiles of an unsplit (N, C, H, W) tensor, halo p
    K, p, N, C, H, W = 3, 1, 2, 3, 6, 5
    Ht = H // K
    X = rng.uniform(-1, 1, (N, C, H, W)).astype(np.float32)
    Xp = np.pad(X, ((0, 0), (0, 0), (p, p), (p, p)))
    out["geom"] = np.array([K, p, N, C, H, W], np.int64)
    out["unsplit"] = X
    # tile r of the packed form = rows r*Ht .. r*Ht + Ht + 2p of the zero-padded unsplit tensor
    packed = np.stack([Xp[:, :, r * Ht:r * Ht + Ht + 2 * p, :] for r in range(K)])
    out["packed"] = packed
    # padded only (zero halo), what the exchange starts from
    padded = np.zeros_like(packed)
    for r in range(K):
        padded[r, :, :, p:p + Ht, p:p + W] = X[:, :, r * Ht:(r + 1) * Ht, :]
    out["padded"] = padded
    # reduce: the adjoint of the exchange on arbitrary padded tiles
    G = rng.standard_normal(packed.shape).astype(np.float32)
    R = G.copy()
    for r in range(K):
        if r + 1 < K:  # my last interior rows receive the lower neighbour's top halo rows
            R[r, :, :, Ht:Ht + p, p:p + W] = G[r, :, :, Ht:Ht + p, p:p + W] + G[r + 1, :, :, 0:p, p:p + W]
        if r > 0:      # my first interior rows receive the upper neighbour's bottom halo rows
            R[r, :, :, p:2 * p, p:p + W] = G[r, :, :, p:2 * p, p:p + W] + G[r - 1, :, :, Ht + p:Ht + 2 * p, p:p + W]
    out["reduce_in"] = G
    out["reduce_out"] = R
    # ---- 3x3 slab convolution, the three passes (float64 on the CPU)
    n, ci, co, h, w = 2, 5, 4, 6, 7
    x = torch.tensor(rng.uniform(-1, 1, (n, ci, h + 2, w + 2)).astype(np.float32), dtype=torch.float64, requires_grad=True)
    wt = torch.tensor((rng.standard_normal((co, ci, 3, 3)) * 0.2).astype(np.float32), dtype=torch.float64, requires_grad=True)
    dy = torch.tensor(rng.standard_normal((n, co, h, w)).astype(np.float32), dtype=torch.float64)
    y = torch.nn.functional.conv2d(x, wt)
    y.backward(dy)
    out["conv_x_pad"] = x.detach().numpy().astype(np.float32)
    out["conv_w"] = wt.detach().numpy().astype(np.float32)
    out["conv_dy"] = dy.numpy().astype(np.float32)
    out["conv_y"] = y.detach().numpy()
    out["conv_dx_pad"] = x.grad.numpy()
    out["conv_dw"] = wt.grad.numpy()
    # ---- the bias of a convolution
    b = rng.uniform(-1, 1, co).astype(np.float32)
    out["bias"] = b
    out["bias_y"] = (out["conv_y"].astype(np.float32) + b[None, :, None, None]).astype(np.float32)  # one fp32 add per element
    out["bias_db"] = dy.numpy().sum(axis=(0, 2, 3))
    # ---- softmax + negative log likelihood, forward and backward (dx += dloss * (y - onehot))
    rows, classes = 4, 10
    logits = (rng.standard_normal((rows, classes)) * 2).astype(np.float32)
    label = rng.integers(0, classes, rows).astype(np.uint32)
    z = logits.astype(np.float64)
    z = z - z.max(axis=1, keepdims=True)
    prob = np.exp(z) / np.exp(z).sum(axis=1, keepdims=True)
    dloss = rng.uniform(0.5, 1.5, rows).astype(np.float32)
    dx0 = rng.standard_normal((rows, classes)).astype(np.float32)
    onehot = np.zeros((rows, classes))
    onehot[np.arange(rows), label] = 1.0
    out["sm_logits"] = logits
    out["sm_label"] = label
    out["sm_y"] = prob
    out["sm_loss"] = -np.log(prob[np.arange(rows), label])
    out["sm_dloss"] = dloss
    out["sm_dx0"] = dx0
    out["sm_dx"] = dx0.astype(np.float64) + dloss[:, None].astype(np.float64) * (prob - onehot)
    np.savez(os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz"), **out)


if __name__ == "__main__":
    main()
