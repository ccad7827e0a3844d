"""Writes the small committed fixtures under tests/golden/.

The reference ships no vectors for this path, so these come from fixed seeds and
the closed form C = A B^T evaluated in numpy int64 (not from the C oracle, which
the fixtures are used to check).  Run from the repo root:
    python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def pack(v):
    u = v.view(np.uint8)
    return np.ascontiguousarray((u[:, 0::2] & 0x0F) | ((u[:, 1::2] & 0x0F) << 4))


def one(m, n, k, seed, name):
    g = torch.Generator().manual_seed(seed)
    a = torch.randint(-8, 8, (m, k), dtype=torch.int8, generator=g).numpy()
    b = torch.randint(-8, 8, (n, k), dtype=torch.int8, generator=g).numpy()
    c = (a.astype(np.int64) @ b.astype(np.int64).T).astype(np.int32)
    np.savez_compressed(os.path.join(HERE, name), a=a, b=b, a_packed=pack(a), b_packed=pack(b), c=c)


if __name__ == "__main__":
    one(32, 48, 64, 0x51AD0000, "gemm_i4_32x48x64.npz")
    one(70, 33, 160, 0x51AD0001, "gemm_i4_70x33x160.npz")
    one(5, 130, 34, 0x51AD0002, "gemm_i4_5x130x34.npz")
