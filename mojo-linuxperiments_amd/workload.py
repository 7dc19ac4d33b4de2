"""Synthetic inputs and shapes of the five workload configurations.

Everything is generated on the host from one integer seed with numpy's
PCG64 generator and uploaded; the GPU never regenerates data, so host libm
and generator details cannot leak into a parity comparison.

The upstream repository has no data files, seeds or fixtures for this path
(its only tests are thread/NUMA closed forms, test_linux_threading.mojo:24-553),
so these generators follow the workload text alone:
  activations ~ N(0,1) with ceil(0.1 % of K) channels scaled by 20,
  weights ~ N(0, 0.02), block Hadamard 128 along K (256 on the 768-wide
  MoE inner dimension), symmetric int8 per token / per output channel.
"""
import math

import numpy as np

HADAMARD_BLOCK = 128
MOE_INNER_BLOCK = 256

# (name, K, N) of the Llama-style 8B projections used by the decode and prefill sweeps
PROJECTIONS = (
    ("qkv", 4096, 6144),
    ("gate", 4096, 14336),
    ("up", 4096, 14336),
    ("down", 14336, 4096),
)
DECODE_BATCHES = (1, 4, 16)
PREFILL_M = 2048

CFG0 = dict(M=32, K=4096, N=4096)
ATTN = dict(B=16, Hq=32, Hkv=8, D=128, T=4096)
MOE = dict(T=512, H=2048, E=128, topk=8, I=768)


def rng(seed, *stream):
    return np.random.default_rng([int(seed), *[int(s) for s in stream]])


def outlier_channels(g, K):
    n = int(math.ceil(0.001 * K))
    return np.sort(g.choice(K, size=n, replace=False))


def activations(seed, M, K, stream=0):
    """fp32 [M,K] ~ N(0,1); ceil(0.001*K) whole channels multiplied by 20."""
    g = rng(seed, 1, stream)
    x = g.standard_normal((M, K), dtype=np.float32)
    ch = outlier_channels(g, K)
    x[:, ch] *= np.float32(20.0)
    return x


def weights(seed, N, K, stream=0, std=0.02):
    """fp32 [N,K] ~ N(0, std), K contiguous."""
    g = rng(seed, 2, stream)
    w = g.standard_normal((N, K), dtype=np.float32)
    w *= np.float32(std)
    return w


def normal(seed, shape, stream=0):
    g = rng(seed, 3, stream)
    return g.standard_normal(shape, dtype=np.float32)


def linear_algorithmic_bytes(M, N, K):
    """HBM bytes one rotated W8A8 linear must move: int8 weights, fp32 x in,
    fp32 y out, both scale vectors."""
    return N * K + 4 * M * K + 4 * M * N + 4 * N + 4 * M


def gemm_ops(M, N, K):
    return 2 * M * N * K


def attention_algorithmic_bytes(B, Hq, Hkv, D, T):
    kv = 2 * B * Hkv * T * D
    scales = 2 * 4 * B * Hkv * T
    qo = 2 * 4 * B * Hq * D
    return kv + scales + qo


def moe_weight_bytes(E, H, I):
    return E * (2 * I * H + H * I)


def moe_ops(T, topk, H, I):
    return T * topk * 2 * (2 * I * H + H * I)
