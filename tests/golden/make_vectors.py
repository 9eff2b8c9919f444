#!/usr/bin/env python3
"""Writes the known-answer vectors under tests/golden/.

The reference ships no fixtures (its bench draws its tensors from clock64() and checks against
cuDNN in the same run, src/openCNN_winograd.cu:221-238,449-480), so these are the definition of
the operation itself, evaluated independently of everything else in this repository: small
integer-valued CHWN inputs and CRSK filters and their 3x3 / pad 1 / stride 1 cross-correlation
in exact int64 arithmetic with numpy only (KHWN).  Every product and sum is exactly
representable in fp32, so a correct fp32 implementation, Winograd or not, must reproduce the
stored outputs bit for bit.

Usage: python tests/golden/make_vectors.py [name ...]   (rewrites the named .npz files next to it,
all of them without arguments)
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

# name -> (N, C, H, W, K, seed)
CASES = {
    "int_n32_c8_h5_w6_k64": (32, 8, 5, 6, 64, 1),      # odd / even sides, one chunk
    "int_n32_c24_h9_w9_k128": (32, 24, 9, 9, 128, 2),  # three chunks, four filter groups
    "int_n33_c5_h4_w7_k40": (33, 5, 4, 7, 40, 3),      # outside the reference's tiling
    # two 16-channel chunks, a 128-filter block: also a shape of the fp16 / bf16 kernels, whose
    # roundings are exact on these values too (|U| <= 18, |V| <= 16)
    "int_n32_c32_h7_w7_k128": (32, 32, 7, 7, 128, 4),
}


def direct_conv_int(x, w):
    """y[k,h,w,n] = sum_{c,r,s} x[c,h+r-1,w+s-1,n] * w[c,r,s,k], zero padding, int64."""
    C, H, W, N = x.shape
    K = w.shape[3]
    xp = np.zeros((C, H + 2, W + 2, N), dtype=np.int64)
    xp[:, 1:H + 1, 1:W + 1, :] = x
    y = np.zeros((K, H, W, N), dtype=np.int64)
    for r in range(3):
        for s in range(3):
            y += np.einsum("chwn,ck->khwn", xp[:, r:r + H, s:s + W, :], w[:, r, s, :].astype(np.int64))
    return y


def main():
    for name, (N, C, H, W, K, seed) in CASES.items():
        if sys.argv[1:] and name not in sys.argv[1:]:
            continue
        rng = np.random.default_rng(seed)
        # multiples of 1/4 would survive G g G^T exactly as well; integers keep the file small
        x = rng.integers(-4, 5, size=(C, H, W, N)).astype(np.int8)
        w = (4 * rng.integers(-2, 3, size=(C, 3, 3, K))).astype(np.int8)  # multiples of 4: U = G g G^T stays integral
        y = direct_conv_int(x.astype(np.int64), w)
        assert np.abs(y).max() < 2 ** 22
        np.savez_compressed(os.path.join(HERE, name + ".npz"), x=x, w=w, y=y.astype(np.int32))
        print(name, x.shape, w.shape, y.shape, "max |y|", int(np.abs(y).max()))


if __name__ == "__main__":
    main()
