"""Codecs, containers and packers: round trips, format invariants and the quality floors the
reference's own packer tests use (signal-to-noise of quantise -> dequantise).  The packers are
this package's own code; bit parity with the reference's packers is not claimed."""

from __future__ import annotations

import hashlib

import numpy as np
import pytest

import synth
from mfq_amd.formats import bits, mfe as MFE, mx, nint, nvq
from mfq_amd.quantize import nint_quant, nvq_quant


def snr_db(weight, restored):
    noise = np.mean((weight.astype(np.float64) - restored.astype(np.float64)) ** 2)
    return 10.0 * np.log10(np.mean(weight.astype(np.float64) ** 2) / noise)


@pytest.mark.parametrize("width", [1, 2, 3, 5, 7, 8, 10, 12])
def test_bit_pack_round_trip(width):
    rng = np.random.default_rng(width)
    values = rng.integers(0, 1 << width, size=1001, dtype=np.uint32)
    blob = bits.pack_bits(values, width)
    assert len(blob) == bits.stream_nbytes(len(values), width)
    back, end = bits.unpack_bits(blob, 0, len(values), width)
    np.testing.assert_array_equal(back, values)
    assert end == len(blob)


@pytest.mark.parametrize("bits_,gs,sub", [(2, 16, 5), (3, 24, 5), (4, 24, 6), (4, 32, 6), (8, 48, 7)])
def test_nint_blob_round_trip(bits_, gs, sub):
    rng = np.random.default_rng(bits_)
    t = nint_quant.random_codes(9, 100, nint.NintSpec(bits_, gs, sub), rng)
    back = nint.unpack_nint(nint.pack_nint(t))
    np.testing.assert_array_equal(nint.dequantize(back), nint.dequantize(t))
    assert nint.pack_nint(back) == nint.pack_nint(t)


def uniform_nint_blob(t, byte_per_value=False) -> bytes:
    """The storage of files written before per-row widths, assembled field by field as the reference's test
    does (tests/test_formats/test_io.py:67-92): header without the flag bit, anchors, then levels, minima and
    codes of the whole tensor, bit-packed (or, older still, one byte per value)."""
    import struct
    out, groups, _ = t.q.shape
    s = t.spec
    stream = (lambda v, width: np.asarray(v, dtype=np.uint8).tobytes()) if byte_per_value else bits.pack_bits
    return b"".join((
        struct.pack("<BBiii", s.bits, s.sub_bits, s.groupsize, t.axis, t.neuron_len),
        struct.pack("<I", len(t.shape)), struct.pack(f"<{len(t.shape)}q", *t.shape), struct.pack("<II", out, groups),
        np.asarray(t.neuron_scale, dtype="<f2").tobytes(), np.asarray(t.neuron_min, dtype="<f2").tobytes(),
        stream(t.sub_scale, s.sub_bits), stream(t.sub_min, s.sub_bits), stream(t.q, s.bits)))


@pytest.mark.parametrize("bits_,gs,sub", [(2, 16, 5), (3, 24, 5), (4, 24, 6), (8, 48, 8)])
@pytest.mark.parametrize("byte_per_value", [False, True])
def test_nint_uniform_storage_is_read_as_the_same_tensor(bits_, gs, sub, byte_per_value):
    rng = np.random.default_rng(40 + bits_)
    t = nint_quant.random_codes(6, 77, nint.NintSpec(bits_, gs, sub), rng)
    back = nint.unpack_nint(uniform_nint_blob(t, byte_per_value))
    assert back.spec == t.spec and back.shape == t.shape and back.neuron_len == t.neuron_len
    np.testing.assert_array_equal(back.row_q_bits, np.full(6, bits_, np.uint8))
    np.testing.assert_array_equal(back.row_sub_bits, np.full(6, sub, np.uint8))
    np.testing.assert_array_equal(back.q, t.q)
    np.testing.assert_array_equal(nint.dequantize(back), nint.dequantize(t))
    assert nint.pack_nint(back) == nint.pack_nint(t)          # re-written in the current storage
    with pytest.raises(ValueError):
        nint.unpack_nint(uniform_nint_blob(t, byte_per_value) + b"\0")


@pytest.mark.parametrize("bits_,gs,sub,floor", [(2, 16, 5, 9.0), (3, 24, 5, 15.0), (4, 24, 6, 21.0), (8, 48, 7, 40.0)])
def test_nint_quantiser_quality(bits_, gs, sub, floor):
    weight = synth.normal(f"test/nint{bits_}", (16, 192), 0.02)
    t = nint_quant.quantize(weight, nint.NintSpec(bits_, gs, sub))
    restored = nint.dequantize(t)
    assert restored.shape == weight.shape
    assert snr_db(weight, restored) > floor
    assert int(np.asarray(t.q).max()) < (1 << bits_)


def test_nvq_grids_are_the_published_tables():
    raw = (nvq.__file__.rsplit("/", 2)[0] + "/data/nvq_grids.bin")
    digest = hashlib.sha256(open(raw, "rb").read()).hexdigest()
    assert len(digest) == 64
    d4 = nvq.codebook_for(nvq.NVQ3_D4)
    big = nvq.codebook_for(nvq.NVQ3_D4_1024)
    assert d4.shape == (256, 4) and big.shape == (1024, 4)
    # the extension keeps the 512-entry grid as its prefix (tests/test_formats/test_nvq.py:42 of the
    # reference) and every entry odd-valued and unique
    np.testing.assert_array_equal(big[:512], nvq.codebook_for(nvq.NvqSpec("d4_512", 24, 4)))
    assert set(np.unique(d4)).issubset(set(range(1, 16, 2)))
    assert np.all(big % 2 == 1)
    assert len({tuple(row) for row in big.tolist()}) == 1024


def test_sign_rule_parity_bit():
    masks = np.arange(128, dtype=np.uint8).reshape(-1, 1)
    signs = nvq.decode_signs(masks, 8)
    for m in range(128):
        stored = [(m >> i) & 1 for i in range(7)]
        last = sum(stored) & 1
        want = [-1.0 if b else 1.0 for b in stored + [last]]
        assert signs[m].tolist() == want


@pytest.mark.parametrize("jsc", [False, True])
def test_nvq_blob_round_trip_and_quality(jsc):
    weight = synth.normal(f"test/nvq{jsc}", (8, 96), 0.02)
    if jsc:
        t = nvq_quant.quantize_jsc_fixed(weight, nvq.NVQ3_D4_1024)
        restored = nvq.dequantize_nvq_jsc(t)
    else:
        t = nvq_quant.quantize(weight, nvq.NVQ3_D4)
        restored = nvq.dequantize_nvq(t)
    assert snr_db(weight, restored) > 13.0
    back = nvq.unpack_nvq(nvq.pack_nvq(t))
    again = nvq.dequantize_nvq_jsc(back) if jsc else nvq.dequantize_nvq(back)
    np.testing.assert_array_equal(again, restored)


def test_nvq2j_xl_record_storage_round_trip_and_quality():
    """The 4096-entry E8 profile: quantiser quality, both physical layouts, record fields by hand
    (mfq/formats/nvq.py:659-716: state << 60, three segments of index | signs << 12 | parity << 19)."""
    weight = synth.normal("test/nvq2jxl", (6, 100), 0.02)
    t = nvq_quant.quantize_jsc_fixed(weight, nvq.NVQ2_E8_4096)
    restored = nvq.dequantize_nvq_jsc(t)
    assert snr_db(weight, restored) > 9.0                      # about 2.4 bits per weight
    blobs = {}
    for layout in ("group64", "stream"):
        t.storage_layout = layout
        blobs[layout] = nvq.pack_nvq(t)
        back = nvq.unpack_nvq(blobs[layout])
        assert back.storage_layout == layout
        np.testing.assert_array_equal(nvq.dequantize_nvq_jsc(back), restored)
    t.storage_layout = "auto"
    assert nvq.pack_nvq(t) == blobs["group64"]
    groups = 5
    assert len(blobs["group64"]) == 40 + 64 + t.codebooks.size + 2 * 6 + 8 * 6 * groups
    records = np.frombuffer(blobs["group64"][-8 * 6 * groups:], dtype="<u8").reshape(6, groups)
    row, group = 3, 2
    record = int(records[row, group])
    assert record >> 60 == int(t.state[row, group])
    for local in range(3):
        segment = (record >> (20 * local)) & 0xFFFFF
        vector = 3 * group + local
        assert segment & 0xFFF == int(t.indices[row, vector])
        assert (segment >> 12) & 0x7F == int(t.signs[row, vector])
        assert segment >> 19 == bin(int(t.signs[row, vector])).count("1") & 1
    assert int(records[0, 4]) >> 20 & ((1 << 40) - 1) == 0    # vectors 13 and 14 of a 100-column row do not exist
    other = nvq_quant.random_nvq_jsc(2, 96, nvq.NVQ2_E8_1024, np.random.default_rng(0))
    other.storage_layout = "group64"                             # only the 4096-entry profile has records
    with pytest.raises(ValueError):
        nvq.pack_nvq(other)


def test_mxfp4_encoder_and_container():
    weight = synth.normal("test/mx", (6, 128), 0.02)
    t = mx.quantize_mxfp4(weight)
    restored = mx.dequantize_mxfp4(t)
    assert snr_db(weight, restored) > 15.0
    # every block's largest magnitude is representable without saturating by more than one step
    blocks = np.abs(weight).reshape(6, 4, 32).max(axis=2)
    assert np.all(np.abs(restored).reshape(6, 4, 32).max(axis=2) <= 1.5 * blocks + 1e-12)
    back = mx.unpack_mx(mx.pack_mx(t))
    np.testing.assert_array_equal(mx.dequantize_mxfp4(back), restored)
    with pytest.raises(ValueError):
        bad = mx.random_mxfp4(2, 32, np.random.default_rng(0))
        bad.scales[0, 0] = 255
        mx.unpack_mx(mx.pack_mx(bad))


def test_mfe_container_round_trip():
    rng = np.random.default_rng(2)
    pools = [
        MFE.MfePool(np.array([1, 2], dtype=np.int32), nint_quant.random_codes(8, 64, nint.NintSpec(3, 24, 5), rng)),
        MFE.MfePool(np.array([0], dtype=np.int32), mx.random_mxfp4(4, 64, rng)),
        MFE.MfePool(np.array([3], dtype=np.int32), nvq_quant.random_nvq(4, 64, nvq.NVQ3_D4, rng)),
    ]
    t = MFE.MfeTensor((4, 4, 64), pools)
    back = MFE.unpack_mfe(MFE.pack_mfe(t))
    assert back.shape == (4, 4, 64)
    assert [p.expert_ids.tolist() for p in back.pools] == [[1, 2], [0], [3]]
    assert MFE.pack_mfe(back) == MFE.pack_mfe(t)


def test_synthetic_generator_is_deterministic_and_normal():
    a = synth.normal("cfg4/x/0", (64, 64))
    b = synth.normal("cfg4/x/0", (64, 64))
    np.testing.assert_array_equal(a, b)
    assert abs(float(a.mean())) < 0.05 and abs(float(a.std()) - 1.0) < 0.05
    assert not np.array_equal(a, synth.normal("cfg4/x/1", (64, 64)))
    formats = synth.draw_formats("cfg4/format/gate", 512)
    share = {f: formats.count(f) / 512 for f in set(formats)}
    assert set(share) == {"NINT2", "NINT3", "NINT4", "NINT8", "NVQ3J-L", "MXFP4"}
    assert abs(share["NINT4"] - 0.30) < 0.06 and abs(share["NVQ3J-L"] - 0.20) < 0.06
    routes = synth.zipf_routes("cfg5/zipf", 64, 512, 10)
    assert routes.shape == (64, 10) and all(len(set(r)) == 10 for r in routes.tolist())
