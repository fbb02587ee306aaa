"""Seeded synthetic inputs of the benchmark configurations.

Everything is drawn from one CPU ``torch.Generator`` so the GPU path and the CPU
oracle see identical bits; callers move the tensors to the device themselves.
"""
from __future__ import annotations

from typing import Dict

import torch


def _gen(seed: int) -> torch.Generator:
    return torch.Generator(device='cpu').manual_seed(int(seed))


def sigmoid_input(seed: int, n: int = 4_096_000) -> torch.Tensor:
    """float32 [n], uniform in [-8, 8]."""
    return torch.rand(n, generator=_gen(seed), dtype=torch.float32) * 16.0 - 8.0


def partition_input(seed: int, n: int = 16_777_216) -> torch.Tensor:
    """int32 [n], uniform in [0, 2^31)."""
    return torch.randint(0, 2 ** 31, (n,), generator=_gen(seed), dtype=torch.int64).to(torch.int32)


def pack_w4(q: torch.Tensor) -> torch.Tensor:
    """uint8 values 0..15 of shape [K, N] -> uint8 [K/2, N]; low nibble = even k."""
    q = q.to(torch.uint8)
    return (q[0::2] | (q[1::2] << 4)).contiguous()


def pack_z4(z: torch.Tensor) -> torch.Tensor:
    """uint8 values 0..15 of shape [G, N] -> uint8 [G, N/2]; low nibble = even n."""
    z = z.to(torch.uint8)
    return (z[:, 0::2] | (z[:, 1::2] << 4)).contiguous()


def pack_gptq(q: torch.Tensor) -> torch.Tensor:
    """values 0..15 of shape [K, N] -> int32 [K/8, N], nibble j of a word = k % 8 == j
    (the layout samples/05_llama2_7b_int4.py:136 unpacks)."""
    K, N = q.shape
    q = q.to(torch.int64).view(K // 8, 8, N)
    word = torch.zeros(K // 8, N, dtype=torch.int64)
    for j in range(8):
        word |= q[:, j, :] << (4 * j)
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word)
    return word.to(torch.int32).contiguous()


def w4_problem(seed: int, M: int, K: int, N: int, group: int = 128) -> Dict[str, torch.Tensor]:
    """int4 group-quantised GEMV/GEMM operands: q, z uniform on 0..15, scales
    uniform in [0.001, 0.02] (fp16), x ~ N(0,1) (fp16)."""
    g = _gen(seed)
    q = torch.randint(0, 16, (K, N), generator=g, dtype=torch.int64).to(torch.uint8)
    z = torch.randint(0, 16, (K // group, N), generator=g, dtype=torch.int64).to(torch.uint8)
    s = (torch.rand(K // group, N, generator=g, dtype=torch.float32) * 0.019 + 0.001).to(torch.float16)
    x = torch.randn(M, K, generator=g, dtype=torch.float32).to(torch.float16)
    return {'q': q, 'z': z, 'x': x, 'scales': s, 'qweight': pack_w4(q), 'qzeros': pack_z4(z)}


def w4_bytes(M: int, K: int, N: int) -> int:
    """Algorithmic bytes of one int4 g128 GEMV/GEMM call: packed weights, fp16
    scale + 4-bit zero per group, x and y in fp16."""
    return K * N // 2 + (K // 128) * N * 5 // 2 + 2 * M * K + 2 * M * N


def gemm_inputs(seed: int, n: int):
    """fp16 A, B of shape [n, n], N(0,1) * 0.02."""
    g = _gen(seed)
    a = (torch.randn(n, n, generator=g, dtype=torch.float32) * 0.02).to(torch.float16)
    b = (torch.randn(n, n, generator=g, dtype=torch.float32) * 0.02).to(torch.float16)
    return a, b
