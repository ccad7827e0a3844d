"""Seeded inputs shared by the parity tests (CPU generation, CPU packing)."""
import numpy as np
import torch

SEED_BASE = 0x51AD0000
C_POISON = 0x7F7F7F7F  # C is pre-filled with this to prove the GEMM overwrites it


def make_values(rows, k, seed, lo=-8, hi=8):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(lo, hi, (rows, k), dtype=torch.int8, generator=g)


def make_operands(m, n, k, seed):
    """int8 value matrices A[m,k], B[n,k], uniform on the inclusive range [-8, 7]."""
    g = torch.Generator().manual_seed(seed)
    a = torch.randint(-8, 8, (m, k), dtype=torch.int8, generator=g)
    b = torch.randint(-8, 8, (n, k), dtype=torch.int8, generator=g)
    return a, b


def pack_cpu(values: torch.Tensor) -> torch.Tensor:
    """Low nibble = even k; numpy bit arithmetic, independent of the library under test."""
    v = values.numpy().view(np.uint8)
    packed = (v[:, 0::2] & 0x0F) | ((v[:, 1::2] & 0x0F) << 4)
    return torch.from_numpy(np.ascontiguousarray(packed).view(np.int8))


def poisoned_c(m, n, device):
    return torch.full((m, n), C_POISON, dtype=torch.int32, device=device)
