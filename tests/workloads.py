"""Seeded synthetic inputs for the five benchmark configurations.

All tensors are generated on the CPU with an explicit ``torch.Generator`` so that the CPU
checker and the GPU kernels see identical bits; callers copy them to the device.

  C1  4096x4096 bf16 ~N(0,1)                           MXFP8 E4M3 round trip
  C2  2^24 fp32 ~N(0,1) + 0.1% x1e4 outliers + 0.1% zeros + 0.1% subnormal-range
  C3  14336x4096 bf16 Student-t(3)*0.02, 0.1% zero blocks, 0.1% blocks with one inf/-inf/NaN
  C4  x [16384,4096] bf16 ~N(0,1), W [14336,4096] bf16 ~N(0,0.02)
  C5  x [4,2048,4096] bf16, gate/up [14336,4096], down [4096,14336] bf16 ~N(0,0.02)
"""
from __future__ import annotations

import torch


def _gen(seed: int) -> torch.Generator:
    return torch.Generator(device="cpu").manual_seed(seed)


def make_c1(rows: int = 4096, cols: int = 4096) -> torch.Tensor:
    return torch.randn(rows, cols, generator=_gen(0)).to(torch.bfloat16)


def make_c2(n: int = 1 << 24) -> torch.Tensor:
    g = _gen(1)
    x = torch.randn(n, generator=g)
    k = max(n // 1000, 1)
    perm = torch.randperm(n, generator=g)
    out_idx, zero_idx, sub_idx = perm[:k], perm[k:2 * k], perm[2 * k:3 * k]
    x[out_idx] *= 1.0e4
    x[zero_idx] = 0.0
    sub_bits = torch.randint(1, 0x7FFFFF, (k,), generator=g, dtype=torch.int32)
    sign = torch.randint(0, 2, (k,), generator=g, dtype=torch.int32) << 31
    x[sub_idx] = (sub_bits | sign).view(torch.float32)
    return x


def make_c3(rows: int = 14336, cols: int = 4096, block: int = 32) -> torch.Tensor:
    g = _gen(2)
    z = torch.randn(rows, cols, generator=g)
    chi2 = torch.zeros(rows, cols)
    for _ in range(3):
        chi2 += torch.randn(rows, cols, generator=g) ** 2
    x = (z / (chi2 / 3.0).sqrt() * 0.02).to(torch.bfloat16)
    del z, chi2
    n_blocks = rows * cols // block
    k = max(n_blocks // 1000, 1)
    perm = torch.randperm(n_blocks, generator=g)
    xb = x.view(n_blocks, block)
    xb[perm[:k]] = 0.0
    sp_blocks = perm[k:2 * k]
    pos = torch.randint(0, block, (k,), generator=g)
    kind = torch.randint(0, 3, (k,), generator=g)
    vals = torch.tensor([float("inf"), float("-inf"), float("nan")], dtype=torch.bfloat16)
    xb[sp_blocks, pos] = vals[kind]
    return x


def make_c4(m: int = 16384, k: int = 4096, n: int = 14336):
    x = torch.randn(m, k, generator=_gen(3)).to(torch.bfloat16)
    w = (0.02 * torch.randn(n, k, generator=_gen(4))).to(torch.bfloat16)
    return x, w


def make_c5(batch: int = 4, seq: int = 2048, hidden: int = 4096, inter: int = 14336):
    x = torch.randn(batch, seq, hidden, generator=_gen(5)).to(torch.bfloat16)
    w_gate = (0.02 * torch.randn(inter, hidden, generator=_gen(6))).to(torch.bfloat16)
    w_up = (0.02 * torch.randn(inter, hidden, generator=_gen(7))).to(torch.bfloat16)
    w_down = (0.02 * torch.randn(hidden, inter, generator=_gen(8))).to(torch.bfloat16)
    return x, w_gate, w_up, w_down
