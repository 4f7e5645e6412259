"""Seeded synthetic inputs for the block-float workloads (shapes follow the reference's models).

Shapes: Falcon-7B MLP 4544/18176 (tt_eager/tt_dnn/op_library/bmm/bmm_op.cpp:779-780), Mistral-7B
4096/14336 with fused QKV 6144 (models/demos/mistral7b/tt/model_config.py:13-18), BERT-Large
384x1024 (bmm_op.cpp:634-693).  Everything is generated on the CPU with numpy's PCG64 so the same
seed gives the same bytes on every host.
"""
from __future__ import annotations

import numpy as np

SEED_BASE = 1234


def f32_to_bf16_bits_rne(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns, round to nearest even (what torch.Tensor.bfloat16() does)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = np.where(nan, (u >> 16) | 0x40, rounded)
    return rounded.astype(np.uint16)


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def normal_tensor(shape, seed: int, scale: float = 1.0) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(scale)).astype(np.float32)


def roundtrip_1k(seed: int = SEED_BASE + 0) -> np.ndarray:
    """fp32 [1,1,1024,1024] ~ N(0,1): the host round trip the reference already runs on CPU."""
    return normal_tensor((1, 1, 1024, 1024), seed)


def stress_mixture(shape=(1, 1, 4096, 4096), seed: int = SEED_BASE + 1) -> np.ndarray:
    """Mixed distribution that stresses the shared exponent.

    One regime per aligned run of 16 elements of a row (= one face row): with p = 0.20 the whole
    run is +0.0.  Otherwise each element is 0.02 * Student-t(df=3) with p = 0.875, or
    N(0,1) * 2**k, k uniform integer in [-20, 20], with p = 0.125.  Overall 70 % / 20 % / 10 %.
    """
    rng = np.random.default_rng(seed)
    n = int(np.prod(shape))
    assert shape[-1] % 16 == 0
    heavy = (0.02 * rng.standard_t(3, size=n)).astype(np.float32)
    wide = (rng.standard_normal(n) * np.exp2(rng.integers(-20, 21, size=n))).astype(np.float32)
    x = np.where(rng.random(n) < 0.875, heavy, wide).astype(np.float32)
    zero_run = rng.random(n // 16) < 0.20
    x.reshape(-1, 16)[zero_run] = 0.0
    return x.reshape(shape)


def activations_bf16(m: int, k: int, seed: int, batch: int | None = None) -> np.ndarray:
    """bf16 bit patterns of N(0,1) activations, shape [m,k] or [batch,m,k]."""
    shape = (m, k) if batch is None else (batch, m, k)
    return f32_to_bf16_bits_rne(normal_tensor(shape, seed))


def weights_f32(k: int, n: int, seed: int, batch: int | None = None) -> np.ndarray:
    shape = (k, n) if batch is None else (batch, k, n)
    return normal_tensor(shape, seed, 0.02)


# name -> (M, K, N, weight format name, batch)
DECODE_FALCON = [("falcon_h_to_4h", 32, 4544, 18176, "bfp8_b", None), ("falcon_4h_to_h", 32, 18176, 4544, "bfp8_b", None)]
DECODE_MISTRAL = [
    ("mistral_qkv", 32, 4096, 6144, "bfp8_b", None),
    ("mistral_o", 32, 4096, 4096, "bfp8_b", None),
    ("mistral_gate", 32, 4096, 14336, "bfp4_b", None),
    ("mistral_up", 32, 4096, 14336, "bfp4_b", None),
    ("mistral_down", 32, 14336, 4096, "bfp4_b", None),
]
# prefill_ff1_256: the same weights under a short prompt (128 <= M < 512 runs on the fused tiled kernel, which expands the
# weights in LDS; from 512 rows on they are expanded to bf16 once per launch)
PREFILL = [("prefill_ff1", 2048, 4096, 14336, "bfp8_b", None), ("bert_bmm", 384, 1024, 1024, "bfp8_b", 12),
           ("prefill_ff1_256", 256, 4096, 14336, "bfp8_b", None)]


def gemm_bytes(m: int, k: int, n: int, fmt: str, batch: int | None = None) -> int:
    """Algorithmic HBM bytes of one block-float GEMM: packed weights + bf16 A + bf16 C."""
    tile = 1088 if fmt == "bfp8_b" else 576
    b = batch or 1
    return b * ((k // 32) * (n // 32) * tile + m * k * 2 + m * n * 2)


def gemm_flops(m: int, k: int, n: int, batch: int | None = None) -> int:
    return 2 * m * k * n * (batch or 1)
