"""Synthetic workloads of the benchmark configurations (used by the tests, bench.py and the smoke run; not part of the
library).

Random numbers come from a counter-based generator that is trivial to restate in any
language: ``splitmix64`` of ``seed + counter`` gives 64 uniform bits; two of them feed a
Box-Muller transform (both normals are used, fp64 math, one rounding to fp32).  Every
tensor has its own seed ``splitmix64(BASE_SEED ^ fnv1a64(tag))``.

Expert formats are drawn per (expert, projection) by inverse CDF over the configured mix.
Weights are either packed from N(0, 0.02^2) draws by this package's packers (``mode="pack"``)
or built from random codes with anchors sized so the dequantised weights have the same
scale (``mode="random"``, the way the reference's kernel tests and CPU fixtures build inputs:
cpp_runtime/tests/make_cpu_quant_fixtures.py:30-57, tests/mixed_family_fixtures.py:49-147).
"""

from __future__ import annotations

import math

import numpy as np

from mfq_amd.formats.mfe import MfePool, MfeTensor
from mfq_amd.formats.mx import Mxfp4Tensor, quantize_mxfp4
from mfq_amd.formats.nint import NINT2, NINT3, NINT4, NINT8, NintSpec, NintTensor
from mfq_amd.formats.nvq import NVQ2_E8_4096, NVQ3_D4, NVQ3_D4_1024, NvqJscTensor, NvqTensor
from mfq_amd.quantize import nint_quant, nvq_quant

BASE_SEED = 20261125
_MASK = (1 << 64) - 1

FORMAT_MIX = (("NINT2", 0.10), ("NINT3", 0.25), ("NINT4", 0.30), ("NINT8", 0.05), ("NVQ3J-L", 0.20), ("MXFP4", 0.10))
NINT_SPECS = {"NINT2": NINT2, "NINT3": NINT3, "NINT4": NINT4, "NINT8": NINT8, "NINT4-32": NintSpec(4, 32, 6)}


def fnv1a64(text: str) -> int:
    h = 0xCBF29CE484222325
    for byte in text.encode("utf-8"):
        h = ((h ^ byte) * 0x100000001B3) & _MASK
    return h


def splitmix64(x):
    """Scalar int or uint64 ndarray."""
    if isinstance(x, np.ndarray):
        with np.errstate(over="ignore"):
            z = x + np.uint64(0x9E3779B97F4A7C15)
            z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
            z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
            return z ^ (z >> np.uint64(31))
    z = (x + 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def tensor_seed(tag: str) -> int:
    return splitmix64(BASE_SEED ^ fnv1a64(tag))


def uniform01(seed: int, count: int, offset: int = 0) -> np.ndarray:
    """fp64 uniforms in (0, 1): (top 53 bits + 0.5) / 2^53."""
    counters = np.arange(offset, offset + count, dtype=np.uint64) + np.uint64(seed & _MASK)
    bits = splitmix64(counters)
    return ((bits >> np.uint64(11)).astype(np.float64) + 0.5) / float(1 << 53)


def normal(tag: str, shape, std: float = 1.0) -> np.ndarray:
    count = int(np.prod(shape))
    pairs = (count + 1) // 2
    u = uniform01(tensor_seed(tag), 2 * pairs)
    radius = np.sqrt(-2.0 * np.log(u[0::2]))
    angle = 2.0 * math.pi * u[1::2]
    z = np.empty(2 * pairs, dtype=np.float64)
    z[0::2] = radius * np.cos(angle)
    z[1::2] = radius * np.sin(angle)
    return (z[:count] * std).astype(np.float32).reshape(shape)


def to_bf16(x: np.ndarray) -> np.ndarray:
    """Round fp32 to bf16 (nearest even), returned as fp32 values."""
    bits = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    rounded = (bits + np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xFFFF0000)
    return rounded.view(np.float32)


def draw_formats(tag: str, experts: int, mix=FORMAT_MIX) -> list[str]:
    u = uniform01(tensor_seed(tag), experts)
    edges = np.cumsum([p for _, p in mix])
    names = [name for name, _ in mix]
    return [names[min(int(np.searchsorted(edges, value, side="right")), len(names) - 1)] for value in u]


def zipf_routes(tag: str, tokens: int, experts: int, top_k: int, s: float = 1.1) -> np.ndarray:
    """``top_k`` distinct experts per token with popularity ~ rank^-s (Gumbel top-k sampling)."""
    logp = -s * np.log(np.arange(1, experts + 1, dtype=np.float64))
    u = uniform01(tensor_seed(tag), tokens * experts).reshape(tokens, experts)
    keys = logp[None, :] - np.log(-np.log(u))
    return np.argsort(-keys, axis=1, kind="stable")[:, :top_k].astype(np.int32)


# ------------------------------------------------------------------ pools --

def pack_weights(fmt: str, weight: np.ndarray):
    if fmt in NINT_SPECS:
        return nint_quant.quantize(weight, NINT_SPECS[fmt])
    if fmt == "NVQ3":
        return nvq_quant.quantize(weight, NVQ3_D4)
    if fmt == "NVQ3J-L":
        return nvq_quant.quantize_jsc_fixed(weight, NVQ3_D4_1024)
    if fmt == "NVQ2J-XL":
        return nvq_quant.quantize_jsc_fixed(weight, NVQ2_E8_4096)
    if fmt == "MXFP4":
        return quantize_mxfp4(weight)
    raise ValueError(f"unknown format {fmt}")


def random_weights(fmt: str, rows: int, width: int, rng: np.random.Generator, std: float = 0.02):
    """Random codes whose dequantised values have standard deviation of the order of ``std``."""
    if fmt in NINT_SPECS:
        spec = NINT_SPECS[fmt]
        ng = -(-width // spec.groupsize)
        K = (1 << spec.sub_bits) - 1
        nmax = spec.nmax
        step = 6.0 * std / max(nmax, 1)            # codes span about +-3 sigma
        return NintTensor(
            spec, (rows, width), 0, rng.integers(0, nmax + 1, (rows, ng, spec.groupsize), dtype=np.uint8),
            np.full(rows, step / K, dtype=np.float32).astype(np.float16).astype(np.float32),
            np.full(rows, 3.0 * std / K, dtype=np.float32).astype(np.float16).astype(np.float32),
            rng.integers(K // 2, K + 1, (rows, ng), dtype=np.uint8),
            rng.integers(K // 2, K + 1, (rows, ng), dtype=np.uint8), width)
    if fmt == "NVQ3":
        t = nvq_quant.random_nvq(rows, width, NVQ3_D4, rng)
        t.neuron_scale[:] = np.float32(np.float16(std / (8.0 * 7.0)))
        return t
    if fmt == "NVQ3J-L":
        t = nvq_quant.random_nvq_jsc(rows, width, NVQ3_D4_1024, rng)
        t.neuron_scale[:] = np.float32(np.float16(std / (4.5 * 56.0)))
        return t
    if fmt == "NVQ2J-XL":
        t = nvq_quant.random_nvq_jsc(rows, width, NVQ2_E8_4096, rng)
        t.neuron_scale[:] = np.float32(np.float16(std / (8.0 * 4.6)))
        return t
    if fmt == "MXFP4":
        log2 = int(math.floor(math.log2(3.0 * std))) - 2
        return Mxfp4Tensor((rows, width), rng.integers(0, 256, (rows, width // 2), dtype=np.uint8),
                           np.full((rows, width // 32), 127 + log2, dtype=np.uint8))
    raise ValueError(f"unknown format {fmt}")


def build_moe_tensor(tag: str, experts: int, out: int, width: int, formats: list[str], mode: str = "random",
                     std: float = 0.02) -> MfeTensor:
    """One logical [experts, out, width] tensor as per-format pools (pool order = first appearance)."""
    order: list[str] = []
    for fmt in formats:
        if fmt not in order:
            order.append(fmt)
    pools = []
    for fmt in order:
        ids = np.array([e for e, f in enumerate(formats) if f == fmt], dtype=np.int32)
        if mode == "pack":
            weight = np.concatenate([normal(f"{tag}/w/{e}", (out, width), std) for e in ids], axis=0)
            tensor = pack_weights(fmt, weight)
        else:
            rng = np.random.default_rng(tensor_seed(f"{tag}/codes/{fmt}") & 0xFFFFFFFF)
            tensor = random_weights(fmt, ids.size * out, width, rng, std)
        pools.append(MfePool(ids, tensor))
    return MfeTensor((experts, out, width), tuple(pools))


def build_layer(tag: str, experts: int, hidden: int, intermediate: int, mix=FORMAT_MIX, mode: str = "random",
                uniform: str | None = None):
    """(gate, up, down) MfeTensors of one MoE layer plus the drawn formats [3][experts]."""
    names = ("gate", "up", "down")
    formats = [[uniform] * experts if uniform else draw_formats(f"{tag}/format/{p}", experts, mix) for p in names]
    gate = build_moe_tensor(f"{tag}/gate", experts, intermediate, hidden, formats[0], mode)
    up = build_moe_tensor(f"{tag}/up", experts, intermediate, hidden, formats[1], mode)
    down = build_moe_tensor(f"{tag}/down", experts, hidden, intermediate, formats[2], mode)
    return (gate, up, down), formats
