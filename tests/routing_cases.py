"""Seeded synthetic routing workloads shared by the tests, the smoke check and the benchmark.

C1..C5 are the five benchmark configurations; inputs are generated on the CPU from
torch.Generator().manual_seed(seed) so that the CPU oracle and the GPU see identical bits.
"""
from dataclasses import dataclass
from typing import Optional

import torch


@dataclass
class Case:
    name: str
    T: int
    H: int
    E: int
    R: int
    K: int
    M: int
    x: torch.Tensor                 # bf16 [T, H]
    topk_idx: torch.Tensor          # int64 [T, K]
    topk_weights: torch.Tensor      # fp32 [T, K]


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def softmax_topk_case(name, T, H, E, R, K, seed=0, M=None) -> Case:
    """x ~ N(0,1) bf16; logits ~ N(0,1); top-K of softmax (unsorted); weights renormalised to sum 1."""
    g = _gen(seed)
    x = torch.randn((T, H), generator=g, dtype=torch.float32).to(torch.bfloat16)
    p = torch.randn((T, E), generator=g, dtype=torch.float32).softmax(dim=-1)
    w, idx = torch.topk(p, K, dim=-1, largest=True, sorted=False)
    w = (w / w.sum(dim=-1, keepdim=True)).contiguous()
    return Case(name, T, H, E, R, K, M or T, x, idx.to(torch.int64).contiguous(), w)


def uniform_topk_case(name, T, H, E, R, K, seed=0, M=None) -> Case:
    """scores = rand(T, E); top-K unsorted; weights = the selected scores."""
    g = _gen(seed)
    x = torch.randn((T, H), generator=g, dtype=torch.float32).to(torch.bfloat16)
    scores = torch.rand((T, E), generator=g, dtype=torch.float32)
    w, idx = torch.topk(scores, K, dim=-1, largest=True, sorted=False)
    return Case(name, T, H, E, R, K, M or T, x, idx.to(torch.int64).contiguous(), w.contiguous())


def skewed_masked_case(name, T, H, E, R, K, seed=0, zipf_s=1.2, masked_ratio=0.05, M=None) -> Case:
    """Gaussian logits + log Zipf(s) bias over a fixed random expert permutation, top-K; then a share of
    the slots is masked to -1 with weight 0."""
    g = _gen(seed)
    x = torch.randn((T, H), generator=g, dtype=torch.float32).to(torch.bfloat16)
    perm = torch.randperm(E, generator=g)
    bias = torch.empty(E, dtype=torch.float32)
    bias[perm] = -zipf_s * torch.log(torch.arange(1, E + 1, dtype=torch.float32))
    logits = torch.randn((T, E), generator=g, dtype=torch.float32) + bias
    w, idx = torch.topk(logits.softmax(dim=-1), K, dim=-1, largest=True, sorted=False)
    mask = torch.rand((T, K), generator=g) < masked_ratio
    idx = idx.masked_fill(mask, -1)
    w = w.masked_fill(mask, 0.0)
    return Case(name, T, H, E, R, K, M or T, x, idx.to(torch.int64).contiguous(), w.contiguous())


def c1(seed=0): return softmax_topk_case("C1", 128, 1024, 8, 2, 2, seed)
def c2(seed=0): return softmax_topk_case("C2", 4096, 2048, 64, 8, 6, seed)
def c3(seed=0): return uniform_topk_case("C3", 8192, 7168, 256, 8, 8, seed)
def c4(seed=0): return skewed_masked_case("C4", 8192, 7168, 256, 8, 8, seed)


def c5_sources(seed=0, R=8, T=128, H=7168, E=256, K=8):
    """Low-latency decode: R logical source ranks of T tokens each, uniform top-K routing."""
    g = _gen(seed)
    x = torch.randn((R, T, H), generator=g, dtype=torch.float32).to(torch.bfloat16)
    scores = torch.rand((R, T, E), generator=g, dtype=torch.float32)
    w, idx = torch.topk(scores, K, dim=-1, largest=True, sorted=False)
    return x, idx.to(torch.int64).contiguous(), w.contiguous()


def small(name, T, H, E, R, K, seed=0, masked_ratio=0.0, M=None) -> Case:
    c = uniform_topk_case(name, T, H, E, R, K, seed, M)
    if masked_ratio > 0:
        g = _gen(seed + 1000)
        mask = torch.rand((T, K), generator=g) < masked_ratio
        c.topk_idx = c.topk_idx.masked_fill(mask, -1)
        c.topk_weights = c.topk_weights.masked_fill(mask, 0.0)
    return c
