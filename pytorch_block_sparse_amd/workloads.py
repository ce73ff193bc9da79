"""Seeded synthetic workloads for tests and benchmarks of the block-sparse linear path.

Every tensor is generated on the CPU from fixed seeds and copied to the device afterwards, so a
CPU checker and the GPU kernels see identical inputs.  Patterns are sampled the way the library
itself samples them (``numpy.random.choice`` without replacement, sorted).
"""
import math
from dataclasses import dataclass

import numpy
import torch

SEED_PATTERN, SEED_VALUES, SEED_X, SEED_DY = 0, 1, 2, 3


@dataclass
class Workload:
    name: str
    in_features: int
    out_features: int
    density: float
    tokens: int
    dtype: torch.dtype
    pattern: str = "uniform"  # or "zipf"
    passes: str = "fwd+dx+dw"  # or "fwd"

    @property
    def grid(self):
        return self.out_features // 32, self.in_features // 32

    @property
    def nnz(self):
        # truncation as in BlockSparseLinear
        return int(self.density * (self.in_features * self.out_features / 1024))

    @property
    def flops_per_gemm(self):
        return 2.0 * self.tokens * self.nnz * 1024

    @property
    def n_gemms(self):
        return 1 if self.passes == "fwd" else 3

    @property
    def algorithmic_bytes_per_gemm(self):
        e = 4 if self.dtype == torch.float32 else 2
        return e * (self.tokens * self.in_features + self.tokens * self.out_features + self.nnz * 1024)


WORKLOADS = {
    "c1_1024x256_d0.1_fp32": Workload("c1_1024x256_d0.1_fp32", 1024, 256, 0.1, 2048, torch.float32, passes="fwd"),
    "c2_768x3072_d0.5_fp32": Workload("c2_768x3072_d0.5_fp32", 768, 3072, 0.5, 4096, torch.float32),
    "c3_3072x768_d0.25_zipf_fp32": Workload("c3_3072x768_d0.25_zipf_fp32", 3072, 768, 0.25, 4096, torch.float32, "zipf"),
    "c4_4096x4096_d0.25_bf16": Workload("c4_4096x4096_d0.25_bf16", 4096, 4096, 0.25, 16384, torch.bfloat16),
    # the headline shape in the reference's own dtype
    "c4_4096x4096_d0.25_fp32": Workload("c4_4096x4096_d0.25_fp32", 4096, 4096, 0.25, 16384, torch.float32),
    # the headline shape at the upper end of the density range the speed-up over dense is asked for
    "c4_4096x4096_d0.5_bf16": Workload("c4_4096x4096_d0.5_bf16", 4096, 4096, 0.5, 16384, torch.bfloat16),
    "c4_4096x4096_d0.5_fp32": Workload("c4_4096x4096_d0.5_fp32", 4096, 4096, 0.5, 16384, torch.float32),
    # the three linear layers patched in every encoder layer of the RoBERTa-base training step
    # (attention.output.dense, intermediate.dense, output.dense) at its 32 x 512 tokens
    "c5_attn_out_768x768_d0.5_fp32": Workload("c5_attn_out_768x768_d0.5_fp32", 768, 768, 0.5, 16384, torch.float32),
    "c5_ffn_in_768x3072_d0.5_fp32": Workload("c5_ffn_in_768x3072_d0.5_fp32", 768, 3072, 0.5, 16384, torch.float32),
    "c5_ffn_out_3072x768_d0.5_fp32": Workload("c5_ffn_out_3072x768_d0.5_fp32", 3072, 768, 0.5, 16384, torch.float32),
}
ROBERTA_LAYER_WORKLOADS = ("c5_attn_out_768x768_d0.5_fp32", "c5_ffn_in_768x3072_d0.5_fp32", "c5_ffn_out_3072x768_d0.5_fp32")


def uniform_positions(X, Y, nnz, seed=SEED_PATTERN):
    """Sorted flat row-major positions of nnz blocks chosen uniformly without replacement."""
    state = numpy.random.get_state()
    try:
        numpy.random.seed(seed)
        pos = numpy.random.choice(X * Y, size=nnz, replace=False)
    finally:
        numpy.random.set_state(state)
    return numpy.sort(pos.astype(numpy.int64))


def zipf_row_counts(X, Y, nnz, exponent=1.2, seed=SEED_PATTERN):
    """Blocks per block-row following rank^-exponent over a seeded permutation of the rows.

    Counts are scaled to sum to nnz, capped at Y with the overflow handed to the next ranks,
    every row keeps at least one block, and rounding is by largest remainder.
    """
    rng = numpy.random.RandomState(seed)
    perm = rng.permutation(X)
    w = numpy.arange(1, X + 1, dtype=numpy.float64) ** (-exponent)
    target = w / w.sum() * nnz
    counts = numpy.zeros(X, dtype=numpy.float64)
    carry = 0.0
    for i in range(X):
        t = target[i] + carry
        c = min(max(t, 1.0), float(Y))
        carry = t - c
        counts[i] = c
    base = numpy.floor(counts).astype(numpy.int64)
    base = numpy.clip(base, 1, Y)
    rem = nnz - int(base.sum())
    order = numpy.argsort(-(counts - numpy.floor(counts)), kind="stable")
    i = 0
    while rem != 0 and i < 10 * X:
        r = order[i % X]
        if rem > 0 and base[r] < Y:
            base[r] += 1
            rem -= 1
        elif rem < 0 and base[r] > 1:
            base[r] -= 1
            rem += 1
        i += 1
    assert rem == 0, "could not distribute blocks"
    out = numpy.zeros(X, dtype=numpy.int64)
    out[perm] = base
    return out


def zipf_positions(X, Y, nnz, exponent=1.2, seed=SEED_PATTERN):
    counts = zipf_row_counts(X, Y, nnz, exponent, seed)
    rng = numpy.random.RandomState(seed + 1000)
    pos = []
    for r in range(X):
        cols = numpy.sort(rng.choice(Y, size=int(counts[r]), replace=False))
        pos.extend(r * Y + cols)
    return numpy.asarray(pos, dtype=numpy.int64)


def make_pattern(w: Workload):
    X, Y = w.grid
    if w.pattern == "zipf":
        pos = zipf_positions(X, Y, w.nnz)
    else:
        pos = uniform_positions(X, Y, w.nnz)
    return [(int(p // Y), int(p % Y)) for p in pos]


def make_inputs(w: Workload, tokens=None):
    """(blocks, data, x, dy) as CPU tensors in w.dtype; data ~ N(0, 1/sqrt(in)), x, dy ~ N(0, 1)."""
    tokens = w.tokens if tokens is None else tokens
    blocks = make_pattern(w)
    g = torch.Generator().manual_seed(SEED_VALUES)
    data = torch.randn((len(blocks) * 32, 32), generator=g) / math.sqrt(w.in_features)
    g = torch.Generator().manual_seed(SEED_X)
    x = torch.randn((tokens, w.in_features), generator=g)
    g = torch.Generator().manual_seed(SEED_DY)
    dy = torch.randn((tokens, w.out_features), generator=g)
    return blocks, data.to(w.dtype), x.to(w.dtype), dy.to(w.dtype)
