"""Synthetic packed pools built directly in device memory, for benchmark-sized layers.

A full 512-expert layer holds 1.6e9 weights; bit-packing that many codes through the
Python codecs would take minutes and tens of GB of host memory.  The benchmark therefore
fills the runtime-layout buffers with random codes on the GPU (torch is used as a random
byte source and allocator only) and hands the library device-pointer descriptors, exactly
as a runtime that already holds the reference loader's buffers would.  Anchors, levels and
scales are chosen so dequantised weights have a standard deviation of the order of 0.02,
which keeps every fp16 stage of the FFN in range.  Random-code inputs are how the
reference's own kernel tests and CPU fixtures exercise these kernels
(cpp_runtime/tests/make_cpu_quant_fixtures.py:30-57).
"""

from __future__ import annotations

import ctypes as C
import math

import numpy as np
import torch

from mfq_amd import _lib as L
from mfq_amd.formats.nint import NintSpec
from mfq_amd.formats.nvq import NVQ3_D4, NVQ3_D4_1024, codebook_for, pack_jsc_tables
from mfq_amd.quantize.nvq_quant import initial_jsc_tables
from synth import NINT_SPECS, tensor_seed


class DevicePool:
    """Device buffers of one pool plus its descriptor; ``arrays`` keeps the tensors alive."""

    def __init__(self, fmt: str, expert_ids: np.ndarray, view: L.Projection, arrays: dict):
        self.fmt, self.expert_ids, self.view, self.arrays = fmt, np.asarray(expert_ids, dtype=np.int32), view, arrays

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.arrays.values())


def _randbytes(n: int, gen: torch.Generator, lo: int = 0, hi: int = 256) -> torch.Tensor:
    return torch.randint(lo, hi, (n,), dtype=torch.uint8, device="cuda", generator=gen)


def device_pool(fmt: str, expert_ids, experts: int, out: int, width: int, seed: int, std: float = 0.02) -> DevicePool:
    n = len(expert_ids)
    rows = n * out
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed & 0x7FFFFFFF)
    local = np.full(experts, -1, dtype=np.int32)
    local[np.asarray(expert_ids)] = np.arange(n, dtype=np.int32)
    arrays = {"expert_local": torch.from_numpy(local).cuda()}
    v = L.Projection()
    v.expert_local = arrays["expert_local"].data_ptr()
    v.local_experts, v.output_rows, v.input_width = n, out, width
    if fmt in NINT_SPECS:
        spec: NintSpec = NINT_SPECS[fmt]
        ng = -(-width // spec.groupsize)
        row_bits = ng * spec.groupsize * spec.bits
        stride = (out * row_bits + 7) // 8 + 8
        K = (1 << spec.sub_bits) - 1
        q = _randbytes(n * stride, gen).view(n, stride)
        q[:, stride - 8:] = 0                                  # the guard bytes of every expert stream
        arrays.update(
            q=q, row_bits=torch.full((rows,), spec.bits, dtype=torch.uint8, device="cuda"),
            offsets=(torch.arange(out, dtype=torch.int64, device="cuda") * row_bits).repeat(n),
            sub_scale=_randbytes(rows * ng, gen, K // 2, K + 1), sub_min=_randbytes(rows * ng, gen, K // 2, K + 1),
            scale=torch.full((rows,), float(np.float16(6.0 * std / max(spec.nmax, 1) / K)), dtype=torch.float32, device="cuda"),
            minimum=torch.full((rows,), float(np.float16(3.0 * std / K)), dtype=torch.float32, device="cuda"))
        v.family = L.FAMILY_NINT
        for i, key in enumerate(("q", "row_bits", "offsets", "sub_scale", "sub_min", "scale", "minimum")):
            v.fields[i] = arrays[key].data_ptr()
        v.sizes[0] = n * stride
        v.groups, v.group_size, v.sub_bits, v.uniform_bits, v.q_expert_stride = ng, spec.groupsize, spec.sub_bits, spec.bits, stride
    elif fmt in ("NVQ3", "NVQ3J-L"):
        jsc = fmt == "NVQ3J-L"
        spec = NVQ3_D4_1024 if jsc else NVQ3_D4
        ng, nvec, nsign = math.ceil(width / 24), math.ceil(width / 4), math.ceil(width / 8)
        sizes = [(rows * nvec * spec.index_bits + 7) // 8, (rows * nsign * 7 + 7) // 8, (rows * ng * 4 + 7) // 8]
        if jsc:
            meta = np.frombuffer(pack_jsc_tables(*initial_jsc_tables(spec)), dtype=np.int8)
            anchor = std / (4.5 * 56.0)
        else:
            meta = np.ascontiguousarray(codebook_for(spec), dtype=np.int8).reshape(-1)
            anchor = std / (8.0 * 7.0)
        arrays.update(
            indices=_randbytes(sizes[0] + 8, gen), signs=_randbytes(sizes[1] + 8, gen), states=_randbytes(sizes[2] + 8, gen),
            anchors=torch.full((rows,), float(np.float16(anchor)), dtype=torch.float32, device="cuda"),
            meta=torch.from_numpy(meta.copy()).cuda())
        v.family = L.FAMILY_NVQ
        for i, key in enumerate(("indices", "signs", "states", "anchors", "meta")):
            v.fields[i] = arrays[key].data_ptr()
        for i in range(3):
            v.sizes[i] = sizes[i]
        v.groups, v.group_size, v.sub_bits, v.format = ng, 24, 4, 15 if jsc else 3
        v.nvec, v.nsign = nvec, nsign
    elif fmt == "MXFP4":
        log2 = int(math.floor(math.log2(3.0 * std))) - 2
        arrays.update(values=_randbytes(rows * width // 2, gen),
                      scales=_randbytes(rows * width // 32, gen, 127 + log2 - 1, 127 + log2 + 2))
        v.family = L.FAMILY_MXFP4
        v.fields[0], v.fields[1] = arrays["values"].data_ptr(), arrays["scales"].data_ptr()
        v.sizes[0], v.sizes[1] = rows * width // 2, rows * width // 32
        v.groups, v.group_size = width // 32, 32
    else:
        raise ValueError(f"unknown format {fmt}")
    return DevicePool(fmt, expert_ids, v, arrays)


class DeviceMoeTensor:
    """One logical [experts, out, width] tensor as device pools (mirrors MixedMoeRuntime)."""

    def __init__(self, tag: str, experts: int, out: int, width: int, formats: list[str]):
        self.experts, self.out_per_expert, self.neuron_len = experts, out, width
        order = []
        for f in formats:
            if f not in order:
                order.append(f)
        self.formats = list(formats)
        self.pools = [device_pool(f, [e for e, g in enumerate(formats) if g == f], experts, out, width,
                                  tensor_seed(f"{tag}/{f}")) for f in order]
        self._views = (L.Projection * len(self.pools))(*[p.view for p in self.pools])
        self.struct = L.MoeTensor(self._views, len(self.pools), experts, out, width)

    def nbytes(self) -> int:
        return sum(p.nbytes() for p in self.pools)

    def pool_of(self, expert: int):
        for pool in self.pools:
            where = np.flatnonzero(pool.expert_ids == expert)
            if where.size:
                return pool, int(where[0])
        raise KeyError(expert)

    def host_layout(self, expert: int) -> dict:
        """Runtime-layout arrays of one expert copied to the host (for the CPU baseline / checks)."""
        pool, l = self.pool_of(expert)
        a, v, out, width = pool.arrays, pool.view, self.out_per_expert, self.neuron_len
        rows = slice(l * out, (l + 1) * out)
        if v.family == L.FAMILY_NINT:
            g = v.groups
            return dict(family=1, packed=a["q"][l].cpu().numpy().copy(), row_bits=a["row_bits"][rows].cpu().numpy().copy(),
                        row_bit_offsets=a["offsets"][rows].cpu().numpy().copy(),
                        group_scale=a["sub_scale"][l * out * g:(l + 1) * out * g].cpu().numpy().copy(),
                        group_min=a["sub_min"][l * out * g:(l + 1) * out * g].cpu().numpy().copy(),
                        row_scale=a["scale"][rows].cpu().numpy().copy(), row_min=a["minimum"][rows].cpu().numpy().copy(),
                        outputs=out, width=width, group_size=v.group_size, groups=g, q_expert_stride=0)
        if v.family == L.FAMILY_NVQ:
            if "host" not in a:
                a["host"] = {k: a[k].cpu().numpy() for k in ("indices", "signs", "states", "anchors", "meta")}
            h = a["host"]
            return dict(family=2, indices=h["indices"][: v.sizes[0]], aux=h["signs"][: v.sizes[1]],
                        states=h["states"][: v.sizes[2]], anchors=h["anchors"], metadata=h["meta"], format=v.format,
                        state_bits=4, sign_mode=0, outputs=out, width=width, row_offset=l * out)
        return dict(family=3, values=a["values"][l * out * width // 2:(l + 1) * out * width // 2].cpu().numpy().copy(),
                    scales=a["scales"][l * out * width // 32:(l + 1) * out * width // 32].cpu().numpy().copy(),
                    outputs=out, width=width)


def device_layer(tag: str, experts: int, hidden: int, intermediate: int, formats):
    gate = DeviceMoeTensor(f"{tag}/gate", experts, intermediate, hidden, formats[0])
    up = DeviceMoeTensor(f"{tag}/up", experts, intermediate, hidden, formats[1])
    down = DeviceMoeTensor(f"{tag}/down", experts, hidden, intermediate, formats[2])
    return gate, up, down
