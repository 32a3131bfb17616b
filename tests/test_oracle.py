"""Pins the CPU oracle: against the reference's own CPU library compiled from its sources
(oracle/_ref, when present), against committed golden vectors written by that library, and
against what the mathematics fixes (closed forms, FP64 decoded-weight sums, brute force)."""

import ctypes as C
from pathlib import Path

import numpy as np
import pytest

from helpers import bits_equal
from mfq_amd.formats import mx as FM, nint as FN, nvq as FV
from mfq_amd.formats.bits import pack_bits, unpack_bits
from mfq_amd.quantize import nint_quant as QN, nvq_quant as QV
from oracle import oracle as O

GOLDEN = Path(__file__).resolve().parent / "golden"
needs_ref = pytest.mark.skipif(O.ref_lib() is None, reason="oracle/_ref not built (reference sources absent)")


# ------------------------------------------------------------------ bits ----
@pytest.mark.parametrize("bits", [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 12])
def test_bitstream_is_little_endian_lsb_first(bits):
    rng = np.random.default_rng(bits)
    values = rng.integers(0, 1 << bits, 1001, dtype=np.uint32)
    nbytes = (values.size * bits + 7) // 8
    out = np.zeros(nbytes, dtype=np.uint8)
    O.lib().orc_pack_bits(values.ctypes.data_as(C.POINTER(C.c_uint32)), values.size, bits,
                          out.ctypes.data_as(C.POINTER(C.c_uint8)), nbytes)
    # closed form: value i occupies bits [i*b, (i+1)*b) == np.packbits(little) of its bit planes
    planes = ((values[:, None] >> np.arange(bits)[None, :]) & 1).astype(np.uint8)
    assert np.array_equal(out, np.packbits(planes.reshape(-1), bitorder="little"))
    assert pack_bits(values, bits) == out.tobytes()
    back, end = unpack_bits(out.tobytes(), 0, values.size, bits)
    assert end == nbytes and np.array_equal(back, values)
    ptr = out.ctypes.data_as(C.POINTER(C.c_uint8))
    for i in (0, 1, 7, 500, 1000):
        assert O.lib().orc_bits_at(ptr, nbytes, i * bits, bits) == values[i]


# ----------------------------------------------------------- conversions ----
def test_half_to_float_exhaustive():
    halves = np.arange(65536, dtype=np.uint16)
    expect = halves.view(np.float16).astype(np.float32)
    got = np.array([O.lib().orc_f16_to_f32(int(h)) for h in halves], dtype=np.float32)
    finite = ~np.isnan(expect)
    assert np.array_equal(got[finite].view(np.uint32), expect[finite].view(np.uint32))
    assert np.isnan(got[~finite]).all()


def test_float_to_half_matches_ieee_rne():
    rng = np.random.default_rng(0)
    halves = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mids = (halves[:-1] + halves[1:]) / 2                      # exact ties
    samples = np.concatenate([halves, mids, np.nextafter(mids, np.inf), np.nextafter(mids, -np.inf),
                              rng.normal(0, 100, 20000), rng.normal(0, 1e-5, 20000), [65504, 65519.99, 65520, 1e9, 2.0**-25,
                                                                                          np.nextafter(2.0**-25, 1), 0.0]])
    samples = np.concatenate([samples, -samples])
    with np.errstate(over="ignore"):
        expect = samples.astype(np.float16).view(np.uint16)
    got = np.array([O.lib().orc_f64_to_f16(float(v)) for v in samples], dtype=np.uint16)
    assert np.array_equal(got, expect)
    f32 = samples.astype(np.float32)
    with np.errstate(over="ignore"):
        expect32 = f32.astype(np.float16).view(np.uint16)
    got32 = np.array([O.lib().orc_f32_to_f16(float(v)) for v in f32], dtype=np.uint16)
    assert np.array_equal(got32, expect32)


def test_bf16_rounding():
    rng = np.random.default_rng(1)
    x = rng.normal(0, 3, 5000).astype(np.float32)
    import torch
    expect = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([O.lib().orc_f32_to_bf16(float(v)) for v in x], dtype=np.uint16)
    assert np.array_equal(got, expect)


# ------------------------------------------------------------------ NINT ----
NINT_SWEEP = [(bits, width, gs) for bits in range(1, 9) for width in (1, 7, 8, 9, 17, 63, 65) for gs in (3, 7, 24, 28, 32, 64)]


def _nint_fixture(bits, rows, width, gs, seed, bit_offset=0):
    """Random-code rows without tail padding and an unaligned first bit, like the reference's
    fixture (cpp_runtime/tests/packed_nint_cpu_test.cpp:34-61)."""
    rng = np.random.default_rng(seed)
    groups = -(-width // gs)
    row_bits = np.array([1 + (bits + r) % 8 for r in range(rows)], dtype=np.uint8) if rows > 1 else np.array([bits], dtype=np.uint8)
    offsets, cursor, pieces = [], bit_offset, [np.zeros(bit_offset, dtype=np.uint8)]
    for r in range(rows):
        codes = rng.integers(0, 1 << int(row_bits[r]), width, dtype=np.uint32)
        offsets.append(cursor)
        pieces.append(((codes[:, None] >> np.arange(int(row_bits[r]))[None, :]) & 1).astype(np.uint8).reshape(-1))
        cursor += width * int(row_bits[r])
    packed = np.packbits(np.concatenate(pieces), bitorder="little")
    packed = np.concatenate([packed, np.zeros(1, dtype=np.uint8)])     # the scalar reader may touch one byte more
    return dict(family=1, packed=packed, row_bits=row_bits, row_bit_offsets=np.array(offsets, dtype=np.int64),
                group_scale=rng.integers(0, 256, rows * groups, dtype=np.uint8),
                group_min=rng.integers(0, 256, rows * groups, dtype=np.uint8),
                row_scale=rng.uniform(1e-4, 1e-3, rows).astype(np.float32),
                row_min=rng.uniform(1e-5, 1e-4, rows).astype(np.float32),
                outputs=rows, width=width, group_size=gs, groups=groups, q_expert_stride=0)


def _fp64_check(y, dense, x):
    """The reference's tolerance: 1e-5 + 2e-6 * sum |terms| (packed_nint_cpu_test.cpp:101-103)."""
    exact = x.astype(np.float64) @ dense.astype(np.float64).T
    bound = 1e-5 + 2e-6 * (np.abs(x.astype(np.float64))[:, None, :] * np.abs(dense.astype(np.float64))[None, :, :]).sum(-1)
    assert np.all(np.abs(y - exact) <= bound)


@pytest.mark.parametrize("bits,width,gs", NINT_SWEEP[::7])
def test_nint_oracle_vs_fp64(bits, width, gs):
    L = _nint_fixture(bits, 5, width, gs, seed=bits * 1000 + width * 10 + gs, bit_offset=3)
    proj = O.Projection(L)
    dense = proj.dequant()
    x = np.random.default_rng(2).uniform(-1, 1, (3, width)).astype(np.float32)
    for order in (0, 1):
        _fp64_check(proj.rows(x, order), dense, x)
    assert np.count_nonzero(proj.rows(np.zeros((2, width), dtype=np.float32))) == 0


@needs_ref
@pytest.mark.parametrize("bits,width,gs", NINT_SWEEP)
def test_nint_oracle_equals_reference_library(bits, width, gs):
    L = _nint_fixture(bits, 6, width, gs, seed=bits * 977 + width * 13 + gs, bit_offset=3)
    proj = O.Projection(L)
    for batch in (1, 7):
        x = np.random.default_rng(batch).uniform(-1, 1, (batch, width)).astype(np.float32)
        assert bits_equal(proj.rows(x, 0), O.ref_nint_matmul(L, x, threads=1, scalar=False))
        assert bits_equal(proj.rows(x, 1), O.ref_nint_matmul(L, x, threads=1, scalar=True))


@needs_ref
@pytest.mark.parametrize("shape", [(640, 2560, FN.NINT4), (2560, 640, FN.NintSpec(5, 28, 7)), (96, 2048, FN.NINT3),
                                   (64, 512, FN.NINT2), (64, 512, FN.NINT8)])
def test_nint_released_geometries_equal_reference(shape):
    n, k, spec = shape
    t = QN.random_codes(n, k, spec, np.random.default_rng(n))
    L = O.nint_runtime(t)
    x = np.random.default_rng(3).uniform(-.15, .15, (3, k)).astype(np.float32)
    assert bits_equal(O.Projection(L).rows(x, 0), O.ref_nint_matmul(L, x, threads=4))
    assert bits_equal(O.Projection(L).dequant(), FN.dequantize(t))


@needs_ref
def test_reference_rejects_what_the_oracle_rejects():
    L = _nint_fixture(4, 3, 17, 7, seed=1)
    assert O.lib().orc_nint_validate(C.byref(O.Projection(L).struct.nint)) == 0
    bad = dict(L, row_bits=np.array([4, 9, 4], dtype=np.uint8))
    assert O.lib().orc_nint_validate(C.byref(O.Projection(bad).struct.nint)) < 0
    with pytest.raises(ValueError):
        O.ref_nint_matmul(bad, np.zeros((1, 17), dtype=np.float32))
    bad = dict(L, row_bit_offsets=np.array([0, 10 ** 9, 0], dtype=np.int64))
    assert O.lib().orc_nint_validate(C.byref(O.Projection(bad).struct.nint)) < 0
    with pytest.raises(ValueError):
        O.ref_nint_matmul(bad, np.zeros((1, 17), dtype=np.float32))


# ------------------------------------------------------------------- NVQ ----
NVQ_CASES = [(FV.NVQ2_E8, False), (FV.NVQ3_D4, False), (FV.NVQ2_E8, True), (FV.NVQ3_D4, True),
             (FV.NVQ3_D4_512, True), (FV.NVQ2_E8_1024, True), (FV.NVQ3_D4_1024, True), (FV.NVQ2_E8_4096, True)]
NVQ_WIDTHS = [1, 4, 7, 8, 9, 23, 24, 25, 47, 48, 49, 96, 250, 2048]


@pytest.mark.parametrize("spec,jsc", NVQ_CASES)
def test_nvq_oracle_dequant_and_fp64(spec, jsc):
    rng = np.random.default_rng(5)
    for width in NVQ_WIDTHS:
        t = (QV.random_nvq_jsc if jsc else QV.random_nvq)(4, width, spec, rng)
        proj = O.Projection(O.nvq_runtime(t))
        dense = proj.dequant()
        assert bits_equal(dense, FV.dequantize_nvq_jsc(t) if jsc else FV.dequantize_nvq(t))
        x = rng.uniform(-1, 1, (7, width)).astype(np.float32)
        for order in (0, 1):
            _fp64_check(proj.rows(x, order), dense, x)


@needs_ref
@pytest.mark.parametrize("spec,jsc", NVQ_CASES)
def test_nvq_oracle_equals_reference_library(spec, jsc):
    rng = np.random.default_rng(6)
    for width in NVQ_WIDTHS:
        for batch in (1, 7):
            t = (QV.random_nvq_jsc if jsc else QV.random_nvq)(5, width, spec, rng)
            L = O.nvq_runtime(t)
            x = rng.uniform(-1, 1, (batch, width)).astype(np.float32)
            assert bits_equal(O.Projection(L).rows(x, 0), O.ref_nvq_rows(L, x)), (spec.codebook, jsc, width, batch)


def test_nvq_loader_alias_of_analytic_nvq3j():
    """Kernel format 11 (bank = state & 1, scale = (state >> 1) + 1; cuda/ops/vq.cpp:214-220, :242-244) is what
    the reference's loader calls an NVQ3J pool whose tables follow the analytic rule: same weights as format 10."""
    rng = np.random.default_rng(12)
    for width in (8, 25, 96, 250):
        t = QV.random_nvq_jsc(5, width, FV.NVQ3_D4, rng)
        L10 = O.nvq_runtime(t)
        L11 = dict(L10, format=11)
        assert bits_equal(O.Projection(L11).dequant(), O.Projection(L10).dequant())
        x = rng.uniform(-1, 1, (3, width)).astype(np.float32)
        assert bits_equal(O.Projection(L11).rows(x, 0), O.Projection(L10).rows(x, 0))
        if O.ref_lib() is not None:
            assert bits_equal(O.Projection(L11).rows(x, 0), O.ref_nvq_rows(L11, x))


def test_nvq_sign_rule_all_masks():
    """Seven stored sign bits, the eighth is their parity: brute force over all 128 masks."""
    spec = FV.NVQ3_D4
    for mask in range(128):
        t = FV.NvqTensor(spec, (1, 8), 0, 8, np.array([1.0], dtype=np.float32), np.array([[1]], dtype=np.uint8),
                         np.array([[3, 9]], dtype=np.uint8), np.array([[mask]], dtype=np.uint8))
        dense = O.Projection(O.nvq_runtime(t)).dequant()[0]
        negative = [(mask >> i) & 1 for i in range(7)]
        negative.append(sum(negative) & 1)
        assert list(np.signbit(dense).astype(int)) == negative
        assert sum(negative) % 2 == 0
        magnitude = np.concatenate([FV.D4_256[3], FV.D4_256[9]]).astype(np.float32)
        assert np.array_equal(np.abs(dense), magnitude)


@needs_ref
def test_scaled_i8_dot_equals_reference():
    rng = np.random.default_rng(8)
    R = O.ref_lib()
    for count in (1, 7, 8, 9, 23, 24):
        w = rng.integers(-127, 128, 24, dtype=np.int8)
        x = rng.uniform(-1, 1, 24).astype(np.float32)
        scale = np.float32(0.0123)
        expect = np.float32(0)
        for i in range(count):                                   # quant_dot.cpp:5-12
            expect = np.float32(expect + np.float32(np.float32(scale * np.float32(w[i])) * x[i]))
        got = R.ref_scaled_i8_dot(w.ctypes.data_as(C.POINTER(C.c_int8)), x.ctypes.data_as(C.POINTER(C.c_float)), count, scale, 1)
        assert np.float32(got) == expect


# ----------------------------------------------------------------- MXFP4 ----
def test_mxfp4_closed_form_exhaustive():
    values = np.tile((np.arange(16, dtype=np.uint8) | (np.arange(16, dtype=np.uint8)[::-1] << 4)), (255, 1))
    t = FM.Mxfp4Tensor((255, 32), values, np.arange(255, dtype=np.uint8).reshape(255, 1))
    dense = O.Projection(O.mxfp4_runtime(t)).dequant()
    grid = [0, .5, 1, 1.5, 2, 3, 4, 6]
    for s in range(255):
        for col in range(32):
            code = (values[s, col // 2] >> (4 * (col & 1))) & 15
            exact = (-1 if code & 8 else 1) * grid[code & 7] * 2.0 ** (s - 127)        # OCP MX closed form
            with np.errstate(over="ignore"):
                expect = np.float32(exact)                                               # 3, 4, 6 x 2^127 overflow fp32
            assert dense[s, col] == expect and np.signbit(dense[s, col]) == bool(code & 8)
    assert bits_equal(dense, FM.dequantize_mxfp4(t))


def test_mxfp4_rows_round_weights_to_half():
    rng = np.random.default_rng(9)
    t = FM.random_mxfp4(6, 64, rng)
    x = rng.uniform(-1, 1, (2, 64)).astype(np.float32)
    dense = FM.dequantize_mxfp4(t).astype(np.float16).astype(np.float32)
    expect = np.zeros((2, 6), dtype=np.float32)
    for b in range(2):
        for r in range(6):
            s = np.float32(0)
            for c in range(64):                                   # cuda/ops/mx.cpp:17-30
                s = np.float32(s + np.float32(x[b, c] * dense[r, c]))
            expect[b, r] = s
    assert bits_equal(O.Projection(O.mxfp4_runtime(t)).rows(x), expect)


# --------------------------------------------------------------- routing ----
def test_expf_accuracy_and_monotonicity():
    xs = np.linspace(-87, 0, 200001).astype(np.float32)
    got = np.array([O.lib().orc_expf(float(v)) for v in xs], dtype=np.float32)
    exact = np.exp(xs.astype(np.float64))
    ulp = np.spacing(exact.astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(got - exact) / ulp) <= 1.5
    assert np.all(np.diff(got) >= 0)
    assert O.lib().orc_expf(0.0) == 1.0 and O.lib().orc_expf(-100.0) == 0.0


@pytest.mark.parametrize("tokens,experts,k", [(8, 512, 10), (5, 40, 4), (3, 1000, 32), (4, 8, 8)])
def test_topk_brute_force(tokens, experts, k):
    rng = np.random.default_rng(experts)
    logits = rng.normal(0, 1.5, (tokens, experts)).astype(np.float32)
    ids, weights = O.topk(logits, k)
    p = np.exp(logits.astype(np.float64) - logits.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    order = np.argsort(-p, axis=-1, kind="stable")[:, :k]
    assert np.array_equal(ids, order)
    chosen = np.take_along_axis(p, order, -1)
    np.testing.assert_allclose(weights, chosen / chosen.sum(-1, keepdims=True), rtol=2e-6)


def test_topk_tie_rule_floor_and_scale():
    logits = np.zeros((2, 64), dtype=np.float32)
    logits[1, 10:14] = 3.0
    ids, weights = O.topk(logits, 6, scale=2.0)
    assert list(ids[0]) == [0, 1, 2, 3, 4, 5]
    assert list(ids[1]) == [10, 11, 12, 13, 0, 1]
    np.testing.assert_allclose(weights.sum(-1), 2.0, rtol=1e-6)
    ids, weights = O.topk(logits, 6, normalize=False)
    np.testing.assert_allclose(weights[0], 1 / 64, rtol=1e-6)
    huge = np.full((1, 8), -1000.0, dtype=np.float32)
    huge[0, 0] = 0
    _, w = O.topk(huge, 2, floor=1e-20)
    assert w[0, 0] == 1.0 and w[0, 1] == 0.0


def test_route_plan_is_bincount_cumsum():
    rng = np.random.default_rng(12)
    ids = rng.integers(0, 37, (53, 5)).astype(np.int32)
    plan = O.route_plan(ids, 37, tile_m=8)
    counts = np.bincount(ids.reshape(-1), minlength=37)
    assert np.array_equal(plan["counts"], counts)
    assert np.array_equal(plan["expert_bounds"], np.concatenate([[0], np.cumsum(counts)]))
    tiles = -(-counts // 8)
    assert np.array_equal(plan["tile_bounds"], np.concatenate([[0], np.cumsum(tiles)]))
    assert np.array_equal(plan["tile_experts"], np.repeat(np.arange(37), tiles))
    flat = ids.reshape(-1)
    assert np.array_equal(flat[plan["ids_dst"]], np.sort(flat, kind="stable"))
    assert np.array_equal(plan["ids_dst"], np.argsort(flat, kind="stable"))


def test_router_logits_order():
    rng = np.random.default_rng(13)
    x = rng.normal(0, 1, (2, 50)).astype(np.float32)
    w = rng.normal(0, 1, (3, 50)).astype(np.float32)
    expect = np.zeros((2, 3), dtype=np.float32)
    for t in range(2):
        for e in range(3):
            s = np.float32(0)
            for c in range(50):
                s = np.float32(s + np.float32(x[t, c] * w[e, c]))
            expect[t, e] = s
    assert bits_equal(O.router_logits(x, w), expect)


# ------------------------------------------------------------ FFN chain ----
def test_swiglu_rounding_chain():
    """half(g) -> half(sigmoid in double) -> half(g*sig) -> half(. * u)  (moe_ffn_pipeline.cpp:154-169)."""
    rng = np.random.default_rng(14)
    g = rng.normal(0, 3, 3000).astype(np.float16)
    u = rng.normal(0, 3, 3000).astype(np.float16)
    sig = (1.0 / (1.0 + np.exp(-g.astype(np.float64)))).astype(np.float16)
    first = (g.astype(np.float32) * sig.astype(np.float32)).astype(np.float16)
    expect = (first.astype(np.float32) * u.astype(np.float32)).astype(np.float16)
    got = np.array([O.lib().orc_swiglu_f16(int(a), int(b), 0.0) for a, b in zip(g.view(np.uint16), u.view(np.uint16))],
                   dtype=np.uint16)
    assert np.array_equal(got, expect.view(np.uint16))


def test_clamped_swiglu_branch():
    """swiglu_limit > 0 (mfq/kernels/cuda/mfe_ffn.h:111-114): g' = min(g, L) (no lower clip), u' = clip(u, -L, L),
    half((g' / (1 + expf(-g'))) * u') in fp32.  Pinned by a float32 numpy closed form to one fp16 step (expf of two
    libraries), and exactly by what the clips imply: an operand beyond the limit gives the result of the limit itself."""
    rng = np.random.default_rng(24)
    g = rng.normal(0, 4, 6000).astype(np.float16)
    u = rng.normal(0, 4, 6000).astype(np.float16)
    one = lambda a, b, limit: O.lib().orc_swiglu_f16(int(np.float16(a).view(np.uint16)), int(np.float16(b).view(np.uint16)), limit)
    for limit in (7.0, 1.5, 0.25):
        L = np.float32(limit)
        gc = np.minimum(g.astype(np.float32), L)
        uc = np.clip(u.astype(np.float32), -L, L)
        act = (gc / (np.float32(1.0) + np.exp(-gc, dtype=np.float32))).astype(np.float32)
        expect = (act * uc).astype(np.float32).astype(np.float16)
        got = O.swiglu_array(g, u, limit)
        a, b = got.view(np.uint16).astype(np.int32), expect.view(np.uint16).astype(np.int32)
        assert np.all(np.abs(a - b) <= 1) and np.mean(a == b) > 0.99
        # the clips, exactly
        assert one(60.0, 3.0, limit) == one(limit, 3.0, limit)
        assert one(2.0, 900.0, limit) == one(2.0, limit, limit) and one(2.0, -900.0, limit) == one(2.0, -limit, limit)
        # no lower clip of the gate: a very negative gate gives (nearly) zero, not -limit * sigmoid(-limit) * u
        assert abs(float(np.uint16(one(-30.0, 1.0, limit)).view(np.float16))) < 1e-6
        # inside the limits it is plain SiLU(g) * u in fp32, one rounding: differs from the table chain only by roundings
        assert one(0.125, 0.125, limit) == one(0.125, 0.125, 1000.0)
    # limit <= 0 selects the table chain
    assert one(1.0, 2.0, 0.0) == one(1.0, 2.0, -1.0)


def test_expert_ffn_composition():
    rng = np.random.default_rng(15)
    gate = O.Projection(O.nint_runtime(QN.random_codes(32, 96, FN.NINT4, rng)))
    up = O.Projection(O.nvq_runtime(QV.random_nvq_jsc(32, 96, FV.NVQ3_D4_1024, rng)))
    down = O.Projection(O.mxfp4_runtime(FM.random_mxfp4(96, 32, rng)))
    x = rng.normal(0, 1, (3, 96)).astype(np.float32)
    got = O.expert_ffn(gate, up, down, x)
    g = gate.rows(x).astype(np.float16)
    u = up.rows(x).astype(np.float16)
    hidden = np.array([[O.lib().orc_swiglu_f16(int(a), int(b), 0.0) for a, b in zip(gr, ur)]
                       for gr, ur in zip(g.view(np.uint16), u.view(np.uint16))], dtype=np.uint16).view(np.float16)
    assert bits_equal(got, down.rows(hidden.astype(np.float32)))


def test_weighted_reduce_order():
    rng = np.random.default_rng(16)
    pairs = rng.normal(0, 1, (2, 10, 8)).astype(np.float16)
    w = rng.uniform(0, 1, (2, 10)).astype(np.float32)
    expect = np.zeros((2, 8), dtype=np.float32)
    for t in range(2):
        for c in range(8):
            s = np.float32(0)
            for r in range(10):
                s = np.float32(s + np.float32(w[t, r] * np.float32(pairs[t, r, c])))
            expect[t, c] = s
    assert bits_equal(O.weighted_reduce(pairs, w), expect)


def test_shared_gate_epilogue_closed_form():
    """The shared-expert epilogue against its definition in float64 (sigmoid from numpy's exp): each output is
    the fp16 rounding of an fp32 value that differs from the float64 one by rounding noise only, so the two
    agree exactly or by one fp16 step; special gates pin the sigmoid itself (0 -> 1/2, large -> 1, -large -> 0)."""
    rng = np.random.default_rng(17)
    tokens, routes, width = 7, 6, 40
    pairs = rng.normal(0, 1, (tokens, routes, width)).astype(np.float16)
    w = rng.uniform(0, 1, (tokens, routes)).astype(np.float32)
    shared = rng.normal(0, 1, (tokens, width)).astype(np.float16)
    gate = rng.normal(0, 3, tokens).astype(np.float32)
    gate[:3] = [0.0, 40.0, -40.0]
    got = O.weighted_reduce_shared_gate(pairs, w, shared, gate)
    routed = O.weighted_reduce(pairs, w).astype(np.float16)
    assert bits_equal(got, O.add_shared_gate(routed, shared, gate))
    sigma = 1.0 / (1.0 + np.exp(-gate.astype(np.float64)))
    exact = routed.astype(np.float64) + sigma[:, None] * shared.astype(np.float64)
    step = np.spacing(np.abs(exact).astype(np.float16)).astype(np.float64)
    assert np.all(np.abs(got.astype(np.float64) - exact) <= 0.5 * step + 1e-6 * np.abs(exact) + 1e-9)
    assert bits_equal(got[0], (routed[0].astype(np.float32) + np.float32(0.5) * shared[0].astype(np.float32)).astype(np.float16))
    assert bits_equal(got[1], (routed[1].astype(np.float32) + shared[1].astype(np.float32)).astype(np.float16))
    assert bits_equal(got[2], routed[2])
    # a transposed operand or a dropped term shows: shared = 0 returns the routed sum, pairs = 0 the gated shared expert
    assert bits_equal(O.weighted_reduce_shared_gate(pairs, w, np.zeros_like(shared), gate), routed)
    only = O.weighted_reduce_shared_gate(np.zeros_like(pairs), w, shared, gate)
    assert bits_equal(only[0], (np.float32(0.5) * shared[0].astype(np.float32)).astype(np.float16))


# --------------------------------------------------------------- golden ----
@pytest.mark.parametrize("name", sorted(p.stem for p in GOLDEN.glob("ref_*.npz")))
def test_oracle_reproduces_reference_golden_vectors(name):
    """Vectors written by tests/golden/make_golden.py from the compiled reference CPU library."""
    data = np.load(GOLDEN / f"{name}.npz", allow_pickle=False)
    layout = {key[2:]: data[key] for key in data.files if key.startswith("L_")}
    for key in ("family", "outputs", "width", "group_size", "groups", "q_expert_stride", "format", "state_bits", "sign_mode"):
        if key in layout:
            layout[key] = int(layout[key])
    proj = O.Projection(layout)
    assert bits_equal(proj.rows(data["x"], 0), data["y_avx2"])
    if "y_scalar" in data.files:
        assert bits_equal(proj.rows(data["x"], 1), data["y_scalar"])


def test_reference_layer_driver_equals_expert_by_expert_rows():
    """ref_layer (one C call per layer: the CPU baseline of bench.py) gives, pair by pair, what the oracle's expert FFN
    gives in the reference's summation order, on the calling thread and on the reference's pinned pool."""
    if O.ref_lib() is None or not hasattr(O.ref_lib(), "ref_layer"):
        pytest.skip("oracle/_ref not built")
    rng = np.random.default_rng(33)
    hidden, inter = 96, 64
    layouts = {}
    for e, kinds in enumerate((("nint", "nvq", "mx"), ("nvq", "mx", "nint"), ("mx", "nint", "nvq"))):
        triple = []
        for which, kind in enumerate(kinds):
            rows, width = (inter, hidden) if which < 2 else (hidden, inter)
            if kind == "nint":
                triple.append(O.nint_runtime(QN.random_codes(rows, width, FN.NINT4, rng)))
            elif kind == "nvq":
                triple.append(O.nvq_runtime(QV.random_nvq_jsc(rows, width, FV.NVQ3_D4_1024, rng)))
            else:
                triple.append(O.mxfp4_runtime(FM.random_mxfp4(rows, width, rng)))
        layouts[e] = tuple(triple)
    x = rng.normal(0, 1, (5, hidden)).astype(np.float32)
    tokens = {0: [0, 3], 1: [1, 2, 4], 2: [4]}
    layer = O.RefLayer(layouts, tokens, x)
    want = np.concatenate([O.expert_ffn(*[O.Projection(L) for L in layouts[e]], x[tokens[e]], order=0) for e in sorted(tokens)])
    for pooled in (False, True):
        got = layer.run(pooled).copy()
        assert bits_equal(got, want), pooled


def test_relu_squared_activation_against_exact_arithmetic():
    """orc_relu2_f16 over every fp16 bit pattern.  The square of an fp16 value has at most 22 significant bits, so it
    is exact in float32 and in float64 alike; rounding the float64 square to fp16 once is therefore the defined
    result (mfq/kernels/cuda/mfe_ffn.h:107-110) reached by a different route."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    up = bits.view(np.float16)
    got = O.relu2_array(up)
    with np.errstate(over="ignore", invalid="ignore"):
        wide = up.astype(np.float64)
        expect = (np.where(wide > 0.0, wide, 0.0) ** 2).astype(np.float16)
    finite = ~np.isnan(up)
    assert np.array_equal(got.view(np.uint16)[finite], expect.view(np.uint16)[finite])
    # negative inputs and both zeros give +0, overflow gives +inf, NaN gives 0 (fmaxf returns the other operand)
    assert got[up < 0].view(np.uint16).max() == 0
    assert np.isinf(got[up == np.float16(300.0)][0])
    assert np.all(got[~finite].view(np.uint16) == 0)


def test_shared_expert_epilogue_special_cases():
    """O.shared_expert_epilogue (mfq/kernels/cuda/mfe_ffn_device.cuh:1249-1263) pinned by what its four operations fix:
    a gate of 0 leaves the fp16-rounded routed sum, a gate of 1 adds the shared row as it is, a shared row of zeros adds
    nothing, the routed sum is rounded to fp16 before the add (a value between two halves moves), and with fp16 gate
    values the product is rounded to fp16 before the add (shared_product_half) while with fp32 gates it is not."""
    routed = np.array([[1.0, 1.0 + 2.0 ** -12, 1000.25, -3.0e-5]], dtype=np.float32)
    shared = np.array([[0.5, -2.0, 3.0, 1.0]], dtype=np.float16)
    rounded = routed.astype(np.float16).astype(np.float32)
    assert rounded[0, 1] != routed[0, 1] and rounded[0, 2] != routed[0, 2]          # the cases do exercise the rounding
    zero_gate = O.shared_expert_epilogue(routed, shared, np.array([0.0], dtype=np.float32))
    assert np.array_equal(zero_gate.view(np.uint32), rounded.view(np.uint32))
    one_gate = O.shared_expert_epilogue(routed, shared, np.array([1.0], dtype=np.float32))
    assert np.array_equal(one_gate, rounded + shared.astype(np.float32))
    no_shared = O.shared_expert_epilogue(routed, np.zeros_like(shared), np.array([0.7], dtype=np.float32))
    assert np.array_equal(no_shared.view(np.uint32), rounded.view(np.uint32))
    # product rounding: 0.3 (fp16 0.30004883) * 3.0 = 0.90014648..., not a half
    gate16 = np.array([0.3], dtype=np.float16)
    exact = float(gate16[0]) * 3.0
    as_half = float(np.float16(exact))
    assert as_half != np.float32(exact)
    half_product = O.shared_expert_epilogue(np.zeros((1, 4), np.float32), shared, gate16)
    float_product = O.shared_expert_epilogue(np.zeros((1, 4), np.float32), shared, gate16.astype(np.float32))
    assert half_product[0, 2] == np.float32(as_half) and float_product[0, 2] == np.float32(exact)
    # independent restatement in float64 (every intermediate is exact in double except the two stated roundings)
    rng = np.random.default_rng(77)
    r = rng.normal(0, 3, (5, 64)).astype(np.float32)
    sh = rng.normal(0, 2, (5, 64)).astype(np.float16)
    g = rng.uniform(0, 1, 5).astype(np.float32)
    want = (r.astype(np.float16).astype(np.float64) + (sh.astype(np.float64) * g.astype(np.float64)[:, None]).astype(np.float32)).astype(np.float32)
    assert np.array_equal(O.shared_expert_epilogue(r, sh, g), want)
