"""Writes the frozen vectors of tests/golden/: seeded bf16-rounded inputs of one small grouped-head case and what
sliding-window 2-simplicial attention gives for them.

The reference holds no vectors for this path (its tests compare two implementations on random inputs,
tests/test_triton.py:9-115), so these come from arithmetic that shares nothing with the oracle's tensor code: the output and
lse from plain Python loops over single (i, j, k) triples in double precision (the definition of
simplicial_attention/triton_two_simplicial_attention.py:148-215: s_ijk = scale * sum_d q_i k1_j k2_k over
i - w1 < j <= i, i - w2 < k <= i, joint softmax, o_i = sum p_ijk v1_j * v2_k), the five gradients from central
differences of those loops (step 1e-5 in double precision).  The tests check every oracle implementation and the HIP
path against the file.

    python tests/golden/make_vectors.py        # rewrites tests/golden/windowed_n20_d32_w9_w4.npz
"""
import math
import os

import numpy as np
import torch

B, N, HQ, HK, D, W1, W2 = 1, 20, 2, 1, 32, 9, 4
NAME = 'windowed_n20_d32_w9_w4.npz'


def forward_loops(q, k1, k2, v1, v2):
    """q (N, HQ, D), the others (N, HK, D), float64 numpy -> out (N, HQ, D), lse (HQ, N)."""
    g = HQ // HK
    scale = D ** -0.5
    out = np.zeros((N, HQ, D))
    lse = np.zeros((HQ, N))
    for h in range(HQ):
        hk = h // g
        for i in range(N):
            logits, pairs = [], []
            for j in range(max(0, i - W1 + 1), i + 1):
                for k in range(max(0, i - W2 + 1), i + 1):
                    logits.append(scale * float(np.sum(q[i, h] * k1[j, hk] * k2[k, hk])))
                    pairs.append((j, k))
            m = max(logits)
            z = sum(math.exp(s - m) for s in logits)
            lse[h, i] = m + math.log(z)
            for s, (j, k) in zip(logits, pairs):
                out[i, h] += math.exp(s - m) / z * v1[j, hk] * v2[k, hk]
    return out, lse


def main():
    gen = torch.Generator().manual_seed(2024)
    draw = lambda h: torch.randn(N, h, D, generator=gen).bfloat16().double().numpy()
    q, k1, k2, v1, v2 = draw(HQ), draw(HK), draw(HK), draw(HK), draw(HK)
    dout = torch.randn(N, HQ, D, generator=gen).bfloat16().double().numpy()
    out, lse = forward_loops(q, k1, k2, v1, v2)
    ins = [q, k1, k2, v1, v2]
    grads = []
    eps = 1e-5
    for x in ins:
        gx = np.zeros_like(x)
        it = np.nditer(x, flags=['multi_index'])
        for _ in it:
            idx = it.multi_index
            keep = x[idx]
            x[idx] = keep + eps
            up = float(np.sum(forward_loops(*ins)[0] * dout))
            x[idx] = keep - eps
            dn = float(np.sum(forward_loops(*ins)[0] * dout))
            x[idx] = keep
            gx[idx] = (up - dn) / (2 * eps)
        grads.append(gx)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), NAME)
    np.savez_compressed(path, shape=np.array([B, N, HQ, HK, D, W1, W2]), q=q, k1=k1, k2=k2, v1=v1, v2=v2, dout=dout, out=out,
                        lse=lse, dq=grads[0], dk1=grads[1], dk2=grads[2], dv1=grads[3], dv2=grads[4])
    print('wrote', path)


if __name__ == '__main__':
    main()
