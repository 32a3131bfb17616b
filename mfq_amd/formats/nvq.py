"""NVQ (neuron-anchored lattice vector quantisation) tensors and their canonical blob.

    w[r, c] = (anchor[r] * S[r, g]) * (+-codeword[index[r, c // dim]][c % dim]),  g = c // 24

``S`` is ``float(sub_scale)`` for the plain profiles (NVQ2/NVQ3) and
``scale_lut[state]`` for the JSC profiles, whose 4-bit group state also selects one
of 1/2/4 int8 codebook banks.  One 7-bit sign mask covers eight weights; the
eighth sign is the parity of the seven stored ones.

Layouts restate mfq/formats/nvq.py (:56-264 tables, :357-371 analytic state tables,
:465-519 JSC header, :791-929 blob).  The three base lattices are byte copies of
llama.cpp's ``kgrid_2bit_256`` / ``kgrid_256`` / ``kgrid_512`` tables and are pinned by
the SHA-256 digests the reference checks at import (mfq/formats/nvq.py:97-101).
"""

from __future__ import annotations

import hashlib
import math
import struct
from dataclasses import dataclass
from pathlib import Path

import numpy as np

from .bits import pack_bits, unpack_bits

_GRID_FILE = Path(__file__).resolve().parent.parent / "data" / "nvq_grids.bin"
_GRID_SHA256 = {
    "e8_256": "915952ebc4af8ddba8113583ca1316fc818843f7b825bbf1a25ae1c39bf0e16d",
    "d4_256": "c9678803c61b2210fbd8cbbb3f965a835409cd7d88a04d086d236261bd221d11",
    "d4_512": "353274c58dd7d8dc5ee960dc8fc54ff9164eaf2b49206b841cd49415cf393f81",
}


def _digits_to_grid(words: np.ndarray, dims: int, digit_bits: int) -> np.ndarray:
    shifts = digit_bits * np.arange(dims, dtype=np.uint32)
    digits = (words.astype(np.uint32)[:, None] >> shifts[None, :]) & ((1 << digit_bits) - 1)
    return np.ascontiguousarray(2 * digits + 1, dtype=np.int8)


def _load_base_grids() -> dict[str, np.ndarray]:
    raw = _GRID_FILE.read_bytes()
    spans = {"e8_256": (0, 512, 8, 2), "d4_256": (512, 1024, 4, 3), "d4_512": (1024, 2048, 4, 3)}
    grids = {}
    for name, (lo, hi, dims, digit_bits) in spans.items():
        chunk = raw[lo:hi]
        if hashlib.sha256(chunk).hexdigest() != _GRID_SHA256[name]:
            raise RuntimeError(f"NVQ lattice table {name} is corrupt")
        grids[name] = _digits_to_grid(np.frombuffer(chunk, dtype="<u2"), dims, digit_bits)
    return grids


def _bit_reverse(values: np.ndarray, bits: int) -> np.ndarray:
    out = np.zeros_like(values)
    work = values.copy()
    for _ in range(bits):
        out = (out << 1) | (work & 1)
        work >>= 1
    return out


def _extend_grid(base: np.ndarray, dims: int, digit_bits: int, entries: int) -> np.ndarray:
    """Nested extension: keep ``base`` and append unused lattice points in
    bit-reversed id order (mfq/formats/nvq.py:223-264)."""
    total_bits = dims * digit_bits
    shifts = digit_bits * np.arange(dims, dtype=np.uint32)
    base_ids = np.bitwise_or.reduce(((base.astype(np.uint32) - 1) // 2) << shifts[None, :], axis=1)
    taken = np.zeros(1 << total_bits, dtype=bool)
    taken[base_ids] = True
    order = _bit_reverse(np.arange(1 << total_bits, dtype=np.uint32), total_bits)
    extra = order[~taken[order]][: entries - base.shape[0]]
    return _digits_to_grid(np.concatenate([base_ids, extra]), dims, digit_bits)


_BASE = _load_base_grids()
E8_256 = _BASE["e8_256"]
D4_256 = _BASE["d4_256"]
D4_512 = _BASE["d4_512"]
E8_1024 = _extend_grid(E8_256, 8, 2, 1024)
E8_4096 = _extend_grid(E8_1024, 8, 2, 4096)
D4_1024 = _extend_grid(D4_512, 4, 3, 1024)

_GRIDS = {"e8_256": E8_256, "e8_1024": E8_1024, "e8_4096": E8_4096,
          "d4_256": D4_256, "d4_512": D4_512, "d4_1024": D4_1024}
_INDEX_BITS = {"e8_256": 8, "e8_1024": 10, "e8_4096": 12, "d4_256": 8, "d4_512": 9, "d4_1024": 10}
_CODEBOOK_ID = {"e8_256": 1, "d4_256": 2, "d4_512": 3, "e8_1024": 4, "e8_4096": 5, "d4_1024": 6}
_ID_CODEBOOK = {v: k for k, v in _CODEBOOK_ID.items()}
# runtime decoder ids (cpp_runtime/backends/cuda/ops/vq.cpp:1047-1075)
_PLAIN_FORMAT = {"e8_256": 2, "d4_256": 3}
_JSC_FORMAT = {"e8_256": 5, "d4_256": 10, "d4_512": 12, "e8_1024": 13, "e8_4096": 14, "d4_1024": 15}

GROUP = 24


@dataclass(frozen=True)
class NvqSpec:
    codebook: str
    groupsize: int = GROUP
    sub_bits: int = 4
    sign_mode: str = "even"

    def __post_init__(self) -> None:
        if self.codebook not in _GRIDS:
            raise ValueError(f"unsupported NVQ codebook: {self.codebook}")
        if self.groupsize <= 0 or self.groupsize % 8:
            raise ValueError("NVQ groupsize must be a positive multiple of 8")
        if not 1 <= self.sub_bits <= 8:
            raise ValueError("NVQ sub_bits must be in [1, 8]")
        if self.sign_mode not in ("even", "index_parity"):
            raise ValueError(f"unsupported NVQ sign mode: {self.sign_mode}")

    @property
    def vector_size(self) -> int:
        return 8 if self.codebook.startswith("e8_") else 4

    @property
    def index_bits(self) -> int:
        return _INDEX_BITS[self.codebook]

    @property
    def codebook_entries(self) -> int:
        return 1 << self.index_bits


NVQ2_E8 = NvqSpec("e8_256")
NVQ3_D4 = NvqSpec("d4_256")
NVQ3_D4_512 = NvqSpec("d4_512")
NVQ3_D4_1024 = NvqSpec("d4_1024")
NVQ2_E8_1024 = NvqSpec("e8_1024")
NVQ2_E8_4096 = NvqSpec("e8_4096")


def codebook_for(spec: NvqSpec) -> np.ndarray:
    return _GRIDS[spec.codebook]


def _geometry(neuron_len: int, spec: NvqSpec) -> tuple[int, int, int]:
    return (math.ceil(neuron_len / spec.groupsize), math.ceil(neuron_len / spec.vector_size),
            math.ceil(neuron_len / 8))


@dataclass
class NvqTensor:
    """Plain NVQ2/NVQ3 tensor (built-in or custom per-matrix codebook)."""
    spec: NvqSpec
    shape: tuple
    axis: int
    neuron_len: int
    neuron_scale: np.ndarray   # [out] f32 (fp16-representable, >= 0)
    sub_scale: np.ndarray      # [out, ng] uint8
    indices: np.ndarray        # [out, nvec]
    signs: np.ndarray          # [out, nsign] 7-bit masks
    codebook: np.ndarray | None = None

    @property
    def runtime_format(self) -> int:
        return _PLAIN_FORMAT[self.spec.codebook]


@dataclass
class NvqJscTensor:
    """NVQ-JSC tensor: 4-bit group state -> (scale_lut, codebook bank)."""
    shape: tuple
    axis: int
    neuron_len: int
    neuron_scale: np.ndarray
    scale_lut: np.ndarray       # [16] f32 (fp16-representable)
    bank_for_state: np.ndarray  # [16] uint8
    state: np.ndarray           # [out, ng] uint8
    indices: np.ndarray
    signs: np.ndarray
    codebooks: np.ndarray       # [banks, entries, dim] int8 in [0, 127]
    base_spec: NvqSpec = NVQ2_E8
    storage_layout: str = "auto"   # "stream", "group64" (NVQ2J-XL only) or "auto" = group64 for NVQ2J-XL

    @property
    def spec(self) -> NvqSpec:
        return self.base_spec

    @property
    def runtime_format(self) -> int:
        return _JSC_FORMAT[self.base_spec.codebook]


def analytic_jsc_state_tables(banks: int, vector_size: int) -> tuple[np.ndarray, np.ndarray]:
    """Deterministic state tables (mfq/formats/nvq.py:357-371)."""
    state = np.arange(16)
    bank = (state % banks).astype(np.uint8)
    if banks == 1:
        scale = state.astype(np.float32)
    elif vector_size == 4:
        scale = (state // banks).astype(np.float32) + 1.0
    else:
        scale = (15.0 * ((state // banks).astype(np.float32) + 1.0) / (16 // banks)).astype(np.float32)
    return scale, bank


def decode_signs(masks: np.ndarray, neuron_len: int, index_parity_bank: np.ndarray | None = None) -> np.ndarray:
    """+-1 per weight from 7-bit masks; bit 7 = parity of the stored seven
    (mfq/quantize/nvq_quant.py:604-620)."""
    masks = np.asarray(masks, dtype=np.uint8)
    lower = (masks[..., None] >> np.arange(7, dtype=np.uint8)) & 1
    last = lower.sum(axis=-1, keepdims=True) & 1
    if index_parity_bank is not None:
        last = last ^ index_parity_bank[..., None]
    negative = np.concatenate([lower, last], axis=-1)
    sign = np.where(negative != 0, np.float32(-1.0), np.float32(1.0))
    return sign.reshape(masks.shape[0], -1)[:, :neuron_len]


def dequantize_nvq(t: NvqTensor) -> np.ndarray:
    """mfq/quantize/nvq_quant.py:623-639."""
    spec = t.spec
    out = t.neuron_scale.size
    table = (codebook_for(spec) if t.codebook is None else t.codebook).astype(np.float32)
    magnitude = table[t.indices].reshape(out, -1)[:, : t.neuron_len]
    bank = None
    if spec.sign_mode == "index_parity":
        bank = ((np.asarray(t.indices) >> 7) & 1).astype(np.uint8)
    sign = decode_signs(t.signs, t.neuron_len, bank)
    group_scale = t.neuron_scale.astype(np.float32)[:, None] * t.sub_scale.astype(np.float32)
    scale = np.repeat(group_scale, spec.groupsize, axis=1)[:, : t.neuron_len]
    return (magnitude * sign) * scale


def dequantize_nvq_jsc(t: NvqJscTensor) -> np.ndarray:
    """mfq/quantize/nvq_jsc.py:1472-1497."""
    spec = t.spec
    out = t.neuron_scale.size
    ng, nvec, _ = _geometry(t.neuron_len, spec)
    per_group = GROUP // spec.vector_size
    padded = np.zeros((out, ng * per_group), dtype=np.int64)
    padded[:, :nvec] = t.indices
    vector_bank = np.repeat(t.bank_for_state[t.state].astype(np.int64), per_group, axis=1)
    magnitude = t.codebooks[vector_bank, padded].reshape(out, -1)[:, : t.neuron_len].astype(np.float32)
    sign = decode_signs(t.signs, t.neuron_len)
    group_scale = t.neuron_scale.astype(np.float32)[:, None] * t.scale_lut.astype(np.float32)[t.state]
    scale = np.repeat(group_scale, GROUP, axis=1)[:, : t.neuron_len]
    return (magnitude * sign) * scale


# ---------------------------------------------------------------- blob ----
_HEADER = struct.Struct("<4sBBHiiI")
_MAGIC = b"NVQ1"
_FLAG_INDEX_PARITY, _FLAG_CUSTOM, _FLAG_JSC = 0x80, 0x40, 0x20
JSC_HEADER_BYTES = 64


def pack_codebook(spec: NvqSpec, codebook: np.ndarray) -> bytes:
    digit_bits = 2 if spec.vector_size == 8 else 3
    digits = (np.asarray(codebook).astype(np.uint16) - 1) // 2
    shifts = (digit_bits * np.arange(spec.vector_size, dtype=np.uint16))[None, :]
    return np.bitwise_or.reduce(digits << shifts, axis=1).astype("<u2").tobytes()


def unpack_codebook(spec: NvqSpec, payload: bytes) -> np.ndarray:
    digit_bits = 2 if spec.vector_size == 8 else 3
    return _digits_to_grid(np.frombuffer(payload, dtype="<u2"), spec.vector_size, digit_bits)


def resolve_jsc_storage_layout(spec: NvqSpec, storage_layout: str = "auto") -> str:
    """Physical layout of the state/index/sign data (mfq/formats/nvq.py:619-642)."""
    layout = ("group64" if spec.codebook == "e8_4096" else "stream") if storage_layout == "auto" else storage_layout
    if layout not in ("stream", "group64"):
        raise ValueError(f"unsupported NVQ-JSC storage layout: {layout}")
    if layout == "group64" and (spec.codebook != "e8_4096" or spec.groupsize != GROUP or spec.sub_bits != 4):
        raise ValueError("NVQ-JSC group64 storage requires NVQ2J-XL")
    return layout


def pack_jsc_group64(state: np.ndarray, indices: np.ndarray, signs: np.ndarray, neuron_len: int) -> bytes:
    """One little-endian 64-bit record per 24-group: ``state << 60`` and three 20-bit segments, each a 12-bit
    index, seven sign bits and their parity; segments past the row's last vector are zero
    (mfq/formats/nvq.py:659-716)."""
    groups, vectors = -(-neuron_len // GROUP), -(-neuron_len // 8)
    state, indices, signs = np.asarray(state), np.asarray(indices), np.asarray(signs)
    out = state.shape[0]
    if state.shape != (out, groups) or indices.shape != (out, vectors) or signs.shape != (out, vectors):
        raise ValueError("group64 streams do not match the tensor geometry")
    if state.max(initial=0) > 15 or indices.max(initial=0) > 4095 or signs.max(initial=0) > 127:
        raise ValueError("group64 values out of range")
    index3 = np.zeros((out, groups * 3), dtype=np.uint64)
    sign3 = np.zeros((out, groups * 3), dtype=np.uint64)
    index3[:, :vectors] = indices
    sign3[:, :vectors] = signs
    parity = np.zeros_like(sign3)
    for bit in range(7):
        parity ^= (sign3 >> np.uint64(bit)) & np.uint64(1)
    segments = (index3 | ((sign3 | (parity << np.uint64(7))) << np.uint64(12))).reshape(out, groups, 3)
    records = state.astype(np.uint64) << np.uint64(60)
    for local in range(3):
        records |= segments[..., local] << np.uint64(20 * local)
    return np.ascontiguousarray(records, dtype="<u8").tobytes()


def _field(planes: np.ndarray, first: int, width: int) -> np.ndarray:
    """Bits [first, first + width) of every record as integers; ``planes`` holds one bit per column, LSB first."""
    weights = (1 << np.arange(width, dtype=np.uint32))
    return planes[..., first:first + width].astype(np.uint32) @ weights


def unpack_jsc_group64(blob, off: int, out: int, neuron_len: int):
    """Inverse of pack_jsc_group64: the records are read as 64 bit planes (the layout of bits.py: LSB first), from
    which the state, the three indices, sign masks and parity bits are sliced by position.  Parity bits and the zero
    padding behind a row's last vector are checked (record layout: mfq/formats/nvq.py:659-716)."""
    groups, vectors = -(-neuron_len // GROUP), -(-neuron_len // 8)
    nbytes = out * groups * 8
    if off + nbytes > len(blob):
        raise ValueError("truncated NVQ-JSC group64 stream")
    raw = np.frombuffer(blob, dtype=np.uint8, count=nbytes, offset=off)
    planes = np.unpackbits(raw, bitorder="little").reshape(out, groups, 64)
    state = _field(planes, 60, 4).astype(np.uint8)
    # segment s of a record covers bits [20 s, 20 s + 20): index (12), sign mask (7), parity of the mask (1)
    segments = planes[..., :60].reshape(out, groups * 3, 20)
    masks = segments[..., 12:19]
    if np.any(segments[..., 19] != (masks.sum(axis=-1) & 1)):
        raise ValueError("invalid NVQ-JSC group64 parity bit")
    if np.any(segments[:, vectors:, :]):
        raise ValueError("NVQ-JSC group64 padding must be zero")
    indices = _field(segments[:, :vectors], 0, 12).astype(np.uint16)
    signs = _field(segments[:, :vectors], 12, 7).astype(np.uint8)
    return state, indices, signs, off + nbytes


def pack_jsc_tables(scale_lut: np.ndarray, bank_for_state: np.ndarray, codebooks: np.ndarray,
                    group64: bool = False) -> bytes:
    """64-byte header (mfq/formats/nvq.py:465-519) + raw int8 banks.  The record storage is marked by
    metadata version 2 and layout byte 1."""
    codebooks = np.ascontiguousarray(codebooks, dtype=np.int8)
    banks, _, dim = codebooks.shape
    if banks not in (1, 2, 4) or codebooks.min() < 0:
        raise ValueError("NVQ-JSC codebooks must be [1|2|4, entries, dim] int8 in [0,127]")
    lut = np.asarray(scale_lut, dtype=np.float32).reshape(16)
    bank_map = np.asarray(bank_for_state, dtype=np.uint8).reshape(16)
    if bank_map.max() >= banks:
        raise ValueError("NVQ-JSC bank_for_state references a missing bank")
    header = bytearray(JSC_HEADER_BYTES)
    header[0], header[1], header[2] = (2 if group64 else 1), banks, 16
    header[52] = 1 if group64 else 0
    analytic_scale, analytic_bank = analytic_jsc_state_tables(banks, dim)
    if np.array_equal(lut, analytic_scale) and np.array_equal(bank_map, analytic_bank):
        header[3] = 1
    header[4:36] = lut.astype("<f2").tobytes()
    header[36:52] = bank_map.tobytes()
    return bytes(header) + codebooks.tobytes()


def _anchors_f16(values: np.ndarray) -> np.ndarray:
    anchors = np.ascontiguousarray(values, dtype="<f2")
    if not np.isfinite(anchors).all() or np.signbit(anchors).any():
        raise ValueError("NVQ neuron anchors must be finite and non-negative in FP16")
    return anchors


def pack_nvq(t) -> bytes:
    spec = t.spec
    out = int(np.asarray(t.neuron_scale).size)
    ng, nvec, nsign = _geometry(t.neuron_len, spec)
    jsc = isinstance(t, NvqJscTensor)
    states = t.state if jsc else t.sub_scale
    if np.asarray(states).shape != (out, ng) or np.asarray(t.indices).shape != (out, nvec) \
            or np.asarray(t.signs).shape != (out, nsign):
        raise ValueError("NVQ stream shapes do not match the tensor geometry")
    profile = _CODEBOOK_ID[spec.codebook]
    tables = b""
    if jsc:
        if spec.groupsize != GROUP or spec.sub_bits != 4 or spec.sign_mode != "even":
            raise ValueError("NVQ-JSC requires gs24, a 4-bit state and parity signs")
        profile |= _FLAG_JSC
        group64 = resolve_jsc_storage_layout(spec, t.storage_layout) == "group64"
        tables = pack_jsc_tables(t.scale_lut, t.bank_for_state, t.codebooks, group64)
        if group64:
            return b"".join([
                _HEADER.pack(_MAGIC, profile, spec.sub_bits, spec.groupsize, t.axis, t.neuron_len, len(t.shape)),
                struct.pack(f"<{len(t.shape)}q", *t.shape), struct.pack("<I", out), tables,
                _anchors_f16(t.neuron_scale).tobytes(), pack_jsc_group64(t.state, t.indices, t.signs, t.neuron_len)])
    else:
        if spec.sign_mode == "index_parity":
            profile |= _FLAG_INDEX_PARITY
        if t.codebook is not None:
            profile |= _FLAG_CUSTOM
            tables = pack_codebook(spec, t.codebook)
    return b"".join([
        _HEADER.pack(_MAGIC, profile, spec.sub_bits, spec.groupsize, t.axis, t.neuron_len, len(t.shape)),
        struct.pack(f"<{len(t.shape)}q", *t.shape),
        struct.pack("<I", out),
        tables,
        _anchors_f16(t.neuron_scale).tobytes(),
        pack_bits(states, spec.sub_bits),
        pack_bits(t.indices, spec.index_bits),
        pack_bits(t.signs, 7),
    ])


def unpack_nvq(blob):
    magic, profile, sub_bits, gs, axis, neuron_len, ndim = _HEADER.unpack_from(blob)
    if magic != _MAGIC:
        raise ValueError(f"invalid NVQ magic: {magic!r}")
    codebook_id = profile & ~(_FLAG_INDEX_PARITY | _FLAG_CUSTOM | _FLAG_JSC)
    if codebook_id not in _ID_CODEBOOK:
        raise ValueError(f"unknown NVQ codebook id: {codebook_id}")
    off = _HEADER.size
    shape = struct.unpack_from(f"<{ndim}q", blob, off)
    off += 8 * ndim
    (out,) = struct.unpack_from("<I", blob, off)
    off += 4
    spec = NvqSpec(_ID_CODEBOOK[codebook_id], gs, sub_bits,
                   "index_parity" if profile & _FLAG_INDEX_PARITY else "even")
    ng, nvec, nsign = _geometry(neuron_len, spec)
    jsc = bool(profile & _FLAG_JSC)
    codebook = lut = bank_map = banks_arr = None
    if jsc:
        header = bytes(blob[off : off + JSC_HEADER_BYTES])
        banks = header[1]
        if header[0] not in (1, 2) or banks not in (1, 2, 4) or header[2] != 16 or any(header[53:64]):
            raise ValueError("unsupported NVQ-JSC metadata header")
        if header[52] != header[0] - 1 or (header[0] == 2 and spec.codebook != "e8_4096"):
            raise ValueError("NVQ-JSC group64 storage requires NVQ2J-XL")
        layout = "group64" if header[0] == 2 else "stream"
        lut = np.frombuffer(header[4:36], dtype="<f2").astype(np.float32)
        bank_map = np.frombuffer(header[36:52], dtype=np.uint8).copy()
        off += JSC_HEADER_BYTES
        nbytes = banks * spec.codebook_entries * spec.vector_size
        banks_arr = np.frombuffer(blob, dtype=np.int8, count=nbytes, offset=off).copy().reshape(
            banks, spec.codebook_entries, spec.vector_size)
        off += nbytes
    elif profile & _FLAG_CUSTOM:
        nbytes = spec.codebook_entries * 2
        codebook = unpack_codebook(spec, bytes(blob[off : off + nbytes]))
        off += nbytes
    anchors = _anchors_f16(np.frombuffer(blob, dtype="<f2", count=out, offset=off)).astype(np.float32)
    off += 2 * out
    if jsc and layout == "group64":
        states, indices, signs, off = unpack_jsc_group64(blob, off, out, neuron_len)
    else:
        states, off = unpack_bits(blob, off, out * ng, sub_bits)
        indices, off = unpack_bits(blob, off, out * nvec, spec.index_bits)
        signs, off = unpack_bits(blob, off, out * nsign, 7)
    if off != len(blob):
        raise ValueError(f"invalid NVQ blob tail: consumed={off}, size={len(blob)}")
    if jsc:
        return NvqJscTensor(tuple(shape), axis, neuron_len, anchors, lut, bank_map, states.reshape(out, ng),
                            indices.reshape(out, nvec), signs.reshape(out, nsign), banks_arr, spec, layout)
    return NvqTensor(spec, tuple(shape), axis, neuron_len, anchors, states.reshape(out, ng),
                     indices.reshape(out, nvec), signs.reshape(out, nsign), codebook)
