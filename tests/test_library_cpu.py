"""The C ABI without a GPU: the library loads, exports every symbol the header declares, its
blob loaders produce the runtime layout the oracle builds from the same tensors, and malformed
input comes back as a status code and a message (never an exception across the boundary)."""

from __future__ import annotations

import ctypes as C
import re
from pathlib import Path

import numpy as np
import pytest

from mfq_amd import _lib as L
from mfq_amd.formats import mfe as MFE, mx, nint, nvq
from mfq_amd.quantize import nint_quant, nvq_quant
from oracle import oracle as O

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "mfq_amd.h").read_text()


def declared_symbols() -> list[str]:
    return sorted(set(re.findall(r"\b(mfq_amd_[a-z0-9_]+)\s*\(", HEADER)))


def test_library_exports_every_declared_symbol():
    lib = L.lib()
    names = declared_symbols()
    assert len(names) >= 25
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/mfq_amd.h but not exported"
    # and the ctypes table binds nothing the header does not declare
    assert set(L.EXPORTS) <= set(names)
    assert lib.mfq_amd_abi_version() >= 1


def test_projection_struct_matches_header_size():
    # 9 pointers + 3 i64 + pointer + 12 i32 (padded) + i64 + 2 i64
    assert C.sizeof(L.Projection) == 9 * 8 + 3 * 8 + 8 + 12 * 4 + 8 + 16


def _host_field(view, index, dtype, count):
    ptr = view.fields[index]
    return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(np.ctypeslib.as_ctypes_type(dtype))), shape=(count,)).copy()


def _load(dtype: str, blob: bytes, out_per_expert: int = 0):
    handle = C.c_void_p()
    buf = (C.c_uint8 * len(blob)).from_buffer_copy(blob)
    status = L.lib().mfq_amd_tensor_load(dtype.encode(), buf, len(blob), out_per_expert, C.byref(handle))
    return status, handle


@pytest.mark.parametrize("bits,gs,sub", [(2, 16, 5), (3, 24, 5), (4, 24, 6), (4, 32, 6), (8, 48, 7)])
def test_nint_loader_matches_oracle_layout(bits, gs, sub):
    rng = np.random.default_rng(bits * 100 + gs)
    t = nint_quant.random_codes(12, 100, nint.NintSpec(bits, gs, sub), rng)
    status, handle = _load("NINT", nint.pack_nint(t), out_per_expert=4)
    assert status == 0, L.lib().mfq_amd_last_error()
    view = L.Projection()
    assert L.lib().mfq_amd_tensor_host_view(handle, C.byref(view)) == 0
    want = O.nint_runtime(t, 4)
    assert (view.family, view.local_experts, view.output_rows, view.input_width) == (1, 3, 4, 100)
    assert (view.groups, view.group_size, view.uniform_bits) == (want["groups"], gs, bits)
    assert view.q_expert_stride == want["q_expert_stride"]
    rows = 12
    np.testing.assert_array_equal(_host_field(view, 0, np.uint8, view.sizes[0]), want["packed"])
    np.testing.assert_array_equal(_host_field(view, 1, np.uint8, rows), want["row_bits"])
    np.testing.assert_array_equal(_host_field(view, 2, np.int64, rows), want["row_bit_offsets"])
    np.testing.assert_array_equal(_host_field(view, 3, np.uint8, rows * view.groups), want["group_scale"].reshape(-1))
    np.testing.assert_array_equal(_host_field(view, 4, np.uint8, rows * view.groups), want["group_min"].reshape(-1))
    np.testing.assert_array_equal(_host_field(view, 5, np.float32, rows), want["row_scale"])
    np.testing.assert_array_equal(_host_field(view, 6, np.float32, rows), want["row_min"])
    # rows of a single-width tensor are regular: the promise uniform_bits makes
    per_row = view.groups * gs * bits
    np.testing.assert_array_equal(want["row_bit_offsets"].reshape(3, 4), np.tile(np.arange(4) * per_row, (3, 1)))
    L.lib().mfq_amd_tensor_free(handle)


@pytest.mark.parametrize("bits,gs,sub", [(2, 16, 5), (3, 24, 5), (4, 24, 6), (8, 48, 7)])
@pytest.mark.parametrize("out_per_expert", [0, 4])
def test_nint_loader_reads_uniform_storage(bits, gs, sub, out_per_expert):
    """A blob without the per-row-width flag (cpp_runtime/backends/cuda/ops/nint.cpp:873-875, :927-958) loads to
    the same runtime layout as the same tensor in the current storage."""
    from test_formats import uniform_nint_blob
    rng = np.random.default_rng(bits * 7 + gs)
    t = nint_quant.random_codes(12, 77, nint.NintSpec(bits, gs, sub), rng)
    views = []
    for blob in (uniform_nint_blob(t), nint.pack_nint(t)):
        status, handle = _load("NINT", blob, out_per_expert)
        assert status == 0, L.lib().mfq_amd_last_error()
        view = L.Projection()
        assert L.lib().mfq_amd_tensor_host_view(handle, C.byref(view)) == 0
        rows, levels = 12, 12 * view.groups
        fields = [_host_field(view, 0, np.uint8, view.sizes[0]), _host_field(view, 1, np.uint8, rows),
                  _host_field(view, 2, np.int64, rows), _host_field(view, 3, np.uint8, levels),
                  _host_field(view, 4, np.uint8, levels), _host_field(view, 5, np.float32, rows),
                  _host_field(view, 6, np.float32, rows)]
        views.append(((view.family, view.local_experts, view.output_rows, view.input_width, view.groups,
                       view.group_size, view.uniform_bits, view.q_expert_stride), fields))
        L.lib().mfq_amd_tensor_free(handle)
    assert views[0][0] == views[1][0]
    for old, new in zip(views[0][1], views[1][1]):
        np.testing.assert_array_equal(old, new)
    status, handle = _load("NINT", uniform_nint_blob(t)[:-1], out_per_expert)
    assert status != 0


@pytest.mark.parametrize("layout", ["group64", "stream"])
def test_nvq2j_xl_loader_reads_both_storages(layout):
    """The 4096-entry E8 profile: 64-bit records per group (metadata version 2) or the three streams; both load
    to the runtime layout the oracle builds, and damaged records are refused
    (cpp_runtime/backends/cuda/ops/vq.cpp:1217-1227, :1319-1361)."""
    rng = np.random.default_rng(23)
    t = nvq_quant.random_nvq_jsc(6, 100, nvq.NVQ2_E8_4096, rng)      # 100 columns: 13 vectors, two padding segments
    t.storage_layout = layout
    blob = nvq.pack_nvq(t)
    status, handle = _load("NVQ", blob)
    assert status == 0, L.lib().mfq_amd_last_error()
    view = L.Projection()
    assert L.lib().mfq_amd_tensor_host_view(handle, C.byref(view)) == 0
    want = O.nvq_runtime(t)
    assert view.family == 2 and view.format == 14 == want["format"]
    assert (view.groups, view.nvec, view.nsign) == (5, 13, 13)
    for index, key in ((0, "indices"), (1, "aux"), (2, "states")):
        got = _host_field(view, index, np.uint8, view.sizes[index])
        np.testing.assert_array_equal(got[: len(want[key])], want[key])
    np.testing.assert_array_equal(_host_field(view, 3, np.float32, 6), want["anchors"])
    got_meta = _host_field(view, 4, np.int8, len(want["metadata"]))
    np.testing.assert_array_equal(got_meta[64:], want["metadata"][64:])           # the banks
    np.testing.assert_array_equal(got_meta[1:52], want["metadata"][1:52])          # banks, states, tables
    L.lib().mfq_amd_tensor_free(handle)
    if layout == "group64":
        tables = 20 + 16 + 4
        records = tables + 64 + t.codebooks.size + 2 * 6

        def refused(at, flip, message):
            bad = bytearray(blob); bad[at] ^= flip
            status, _ = _load("NVQ", bytes(bad))
            assert status != 0 and message in L.lib().mfq_amd_last_error().decode(), L.lib().mfq_amd_last_error()

        refused(records + 2, 0x08, "parity")            # bit 19 of the first record: the parity bit of segment 0
        refused(records + 8 * 4 + 3, 0x10, "padding")   # group 4 of row 0 holds vectors 12..14; 13 and 14 are padding
        refused(tables + 52, 0x01, "group64")            # version 2 without the layout byte
        other = nvq_quant.random_nvq_jsc(4, 96, nvq.NVQ2_E8_1024, rng)
        bad = bytearray(nvq.pack_nvq(other)); bad[tables] = 2; bad[tables + 52] = 1
        status, _ = _load("NVQ", bytes(bad))
        assert status != 0 and "group64" in L.lib().mfq_amd_last_error().decode()


@pytest.mark.parametrize("spec,jsc", [(nvq.NVQ3_D4, False), (nvq.NVQ3_D4_1024, True)])
def test_nvq_loader_matches_oracle_layout(spec, jsc):
    rng = np.random.default_rng(7)
    t = nvq_quant.random_nvq_jsc(6, 96, spec, rng) if jsc else nvq_quant.random_nvq(6, 96, spec, rng)
    status, handle = _load("NVQ", nvq.pack_nvq(t))
    assert status == 0, L.lib().mfq_amd_last_error()
    view = L.Projection()
    assert L.lib().mfq_amd_tensor_host_view(handle, C.byref(view)) == 0
    want = O.nvq_runtime(t)
    assert view.family == 2 and view.format == want["format"]
    assert (view.groups, view.nvec, view.nsign) == (4, 24, 12)
    for index, key in ((0, "indices"), (1, "aux"), (2, "states")):
        got = _host_field(view, index, np.uint8, view.sizes[index])
        np.testing.assert_array_equal(got[: len(want[key])], want[key])
    np.testing.assert_array_equal(_host_field(view, 3, np.float32, 6), want["anchors"])
    np.testing.assert_array_equal(_host_field(view, 4, np.int8, len(want["metadata"])), want["metadata"])
    L.lib().mfq_amd_tensor_free(handle)


def test_nvq_loader_validation_rules_of_the_reference():
    """Malformed NVQ payloads the reference's reader refuses (cpp_runtime/backends/cuda/ops/vq.cpp:1120-1270):
    analytic state tables that do not hold the promised values, an all-zero codeword, index-parity signs on a
    D4 profile, a state that names a missing bank."""
    rng = np.random.default_rng(21)
    t = nvq_quant.random_nvq_jsc(4, 96, nvq.NVQ3_D4_1024, rng)
    good = bytearray(nvq.pack_nvq(t))
    tables = 20 + 16 + 4                  # fixed header, two dimensions, row count
    assert good[tables] == 1 and good[tables + 2] == 16
    status, handle = _load("NVQ", bytes(good))
    assert status == 0, L.lib().mfq_amd_last_error()
    L.lib().mfq_amd_tensor_free(handle)

    def refused(blob, message):
        status, _ = _load("NVQ", bytes(blob))
        assert status != 0 and message in L.lib().mfq_amd_last_error().decode(), L.lib().mfq_amd_last_error()

    if good[tables + 3] == 1:              # analytic mode: any other table value is a contradiction
        bad = bytearray(good); bad[tables + 4 + 2 * 5] ^= 0x01
        refused(bad, "analytic")
        bad = bytearray(good); bad[tables + 36 + 1] = (bad[tables + 36 + 1] + 1) % good[tables + 1]
        if good[tables + 1] > 1:
            refused(bad, "analytic")
    bad = bytearray(good); bad[tables + 36 + 2] = good[tables + 1]
    refused(bad, "missing bank")
    bad = bytearray(good); bad[tables + 64 + 4 * 7 : tables + 64 + 4 * 8] = bytes(4)
    refused(bad, "all zero")
    bad = bytearray(good); bad[tables + 64 + 9] = 200
    refused(bad, "int8")
    bad = bytearray(good); bad[tables + 60] = 1
    refused(bad, "reserved")
    plain = bytearray(nvq.pack_nvq(nvq_quant.random_nvq(4, 96, nvq.NVQ3_D4, rng)))
    plain[4] |= 0x80
    refused(plain, "index parity")


def test_mxfp4_loader_and_nan_scale_rejected():
    rng = np.random.default_rng(3)
    t = mx.random_mxfp4(5, 64, rng)
    status, handle = _load("MXFP4", mx.pack_mx(t))
    assert status == 0
    view = L.Projection()
    assert L.lib().mfq_amd_tensor_host_view(handle, C.byref(view)) == 0
    np.testing.assert_array_equal(_host_field(view, 0, np.uint8, 5 * 32), np.asarray(t.values).reshape(-1))
    np.testing.assert_array_equal(_host_field(view, 1, np.uint8, 5 * 2), np.asarray(t.scales).reshape(-1))
    L.lib().mfq_amd_tensor_free(handle)
    bad = mx.random_mxfp4(2, 32, rng)
    bad.scales[0, 0] = 255                     # E8M0 NaN
    status, handle = _load("MXFP4", mx.pack_mx(bad))
    assert status == L.ERR_INVALID and b"" != L.lib().mfq_amd_last_error()
    for at in (4, 5, 6, 7):                    # version, element kind, reserved (cpp_runtime/backends/cuda/ops/mx.cpp:376-381)
        blob = bytearray(mx.pack_mx(t)); blob[at] ^= 1
        assert _load("MXFP4", bytes(blob))[0] == L.ERR_INVALID


@pytest.mark.parametrize("cut", [0, 3, 17, -1])
def test_truncated_blobs_are_rejected(cut):
    rng = np.random.default_rng(11)
    blob = nint.pack_nint(nint_quant.random_codes(4, 48, nint.NintSpec(4, 24, 6), rng))
    broken = blob[:cut] if cut >= 0 else blob + b"\0"
    status, _ = _load("NINT", broken)
    assert status == L.ERR_INVALID
    assert len(L.lib().mfq_amd_last_error()) > 0
    status, _ = _load("NOPE", blob)
    assert status in (L.ERR_INVALID, L.ERR_UNSUPPORTED)


def test_mfe_container_round_trip_through_the_c_reader():
    rng = np.random.default_rng(5)
    experts, out, width = 6, 4, 96
    pools = [
        MFE.MfePool(np.array([0, 3], dtype=np.int32), nint_quant.random_codes(2 * out, width, nint.NintSpec(4, 24, 6), rng)),
        MFE.MfePool(np.array([1, 4, 5], dtype=np.int32), nvq_quant.random_nvq_jsc(3 * out, width, nvq.NVQ3_D4_1024, rng)),
        MFE.MfePool(np.array([2], dtype=np.int32), mx.random_mxfp4(out, width, rng)),
    ]
    blob = MFE.pack_mfe(MFE.MfeTensor((experts, out, width), pools))
    handle = C.c_void_p()
    buf = (C.c_uint8 * len(blob)).from_buffer_copy(blob)
    assert L.lib().mfq_amd_mfe_load(buf, len(blob), C.byref(handle)) == 0, L.lib().mfq_amd_last_error()
    e, o, w, n = C.c_int32(), C.c_int32(), C.c_int32(), C.c_int32()
    assert L.lib().mfq_amd_mfe_info(handle, C.byref(e), C.byref(o), C.byref(w), C.byref(n)) == 0
    assert (e.value, o.value, w.value, n.value) == (experts, out, width, 3)
    seen = []
    for i in range(3):
        tensor, ids, count = C.c_void_p(), C.c_void_p(), C.c_int32()
        assert L.lib().mfq_amd_mfe_pool(handle, i, C.byref(tensor), C.byref(ids), C.byref(count)) == 0
        values = C.cast(ids, C.POINTER(C.c_int32))
        seen.append([values[j] for j in range(count.value)])
    assert seen == [[0, 3], [1, 4, 5], [2]]
    L.lib().mfq_amd_mfe_free(handle)


def _mfe_bytes(magic, shape, pools, labels=None, short=False):
    """A container assembled by hand: header, then per pool its header, expert ids, dtype label and payload
    (cpp_runtime/backends/cuda/ops/moe.cpp:43-111; "NIM1" pools: count and payload size only, NINT implied)."""
    import struct
    parts = [struct.pack("<4sIIII", magic, *shape, len(pools))]
    for index, (ids, payload) in enumerate(pools):
        ids = np.asarray(ids, dtype="<i4")
        if short:
            parts += [struct.pack("<IQ", ids.size, len(payload)), ids.tobytes(), payload]
        else:
            label = labels[index].encode("ascii")
            parts += [struct.pack("<IIQQ", ids.size, len(label), len(payload), 0), ids.tobytes(), label, payload]
    return b"".join(parts)


def _mfe_status(blob):
    handle = C.c_void_p()
    buf = (C.c_uint8 * len(blob)).from_buffer_copy(blob)
    status = L.lib().mfq_amd_mfe_load(buf, len(blob), C.byref(handle))
    pools = C.c_int32()
    if status == 0:
        assert L.lib().mfq_amd_mfe_info(handle, None, None, None, C.byref(pools)) == 0
        L.lib().mfq_amd_mfe_free(handle)
    return status, pools.value


def test_mfe_older_magics_and_profile_labels_are_read_by_both_readers():
    from test_formats import uniform_nint_blob
    rng = np.random.default_rng(11)
    out, width = 4, 96
    a = nint_quant.random_codes(2 * out, width, nint.NintSpec(4, 24, 6), rng)
    b = nvq_quant.random_nvq_jsc(out, width, nvq.NVQ3_D4_1024, rng)
    c = nint_quant.random_codes(out, width, nint.NintSpec(3, 24, 5), rng)
    shape = (3, out, width)
    pools = [([0, 2], nint.pack_nint(a)), ([1], nvq.pack_nvq(b))]
    for magic, labels in ((b"MFE1", ["NINT", "NVQ"]), (b"NIM2", ["NINTv2", "NVQ3J-L"]), (b"MFE1", ["NINT4", "NVQ3J-L"])):
        blob = _mfe_bytes(magic, shape, pools, labels)
        assert _mfe_status(blob) == (0, 2), L.lib().mfq_amd_last_error()
        back = MFE.unpack_mfe(blob)
        np.testing.assert_array_equal(nint.dequantize(back.pools[0].tensor), nint.dequantize(a))
        np.testing.assert_array_equal(nvq.dequantize_nvq_jsc(back.pools[1].tensor), nvq.dequantize_nvq_jsc(b))
    # the oldest container: NINT pools in the uniform storage, no dtype label
    old = _mfe_bytes(b"NIM1", (3, out, width), [([0, 2], uniform_nint_blob(a)), ([1], uniform_nint_blob(
        nint_quant.random_codes(out, width, nint.NintSpec(4, 24, 6), rng)))], short=True)
    assert _mfe_status(old) == (0, 2), L.lib().mfq_amd_last_error()
    np.testing.assert_array_equal(nint.dequantize(MFE.unpack_mfe(old).pools[0].tensor), nint.dequantize(a))
    del c


def test_mfe_delta_and_uncovered_experts_are_rejected_by_both_readers():
    rng = np.random.default_rng(12)
    out, width = 4, 96
    a = nint_quant.random_codes(2 * out, width, nint.NintSpec(4, 24, 6), rng)
    pools = [([0, 2], nint.pack_nint(a))]
    for blob, message in ((_mfe_bytes(b"MFD1", (2, out, width), [([0, 1], nint.pack_nint(a))], ["NINT"]), "delta"),
                          (_mfe_bytes(b"NID2", (2, out, width), [([0, 1], nint.pack_nint(a))], ["NINT"]), "delta"),
                          (_mfe_bytes(b"MFE1", (3, out, width), pools, ["NINT"]), "cover"),        # expert 1 unowned
                          (_mfe_bytes(b"MFE1", (3, out, width), [([0, 0], nint.pack_nint(a))], ["NINT"]), "unique"),
                          (_mfe_bytes(b"MFEX", (2, out, width), [([0, 1], nint.pack_nint(a))], ["NINT"]), "magic")):
        status, _ = _mfe_status(blob)
        assert status != 0
        assert message in L.lib().mfq_amd_last_error().decode()
        with pytest.raises(ValueError):
            MFE.unpack_mfe(blob)


@pytest.mark.parametrize("name,entries,dim", [("e8_256", 256, 8), ("d4_256", 256, 4), ("d4_512", 512, 4), ("d4_1024", 1024, 4)])
def test_builtin_grids_equal_python_tables(name, entries, dim):
    out = np.zeros(entries * dim, dtype=np.int8)
    n, d = C.c_int32(), C.c_int32()
    status = L.lib().mfq_amd_nvq_grid(name.encode(), out.ctypes.data_as(C.c_void_p), out.size, C.byref(n), C.byref(d))
    assert status == 0 and (n.value, d.value) == (entries, dim)
    spec = nvq.NvqSpec(name, 24, 4)
    np.testing.assert_array_equal(out.reshape(entries, dim), nvq.codebook_for(spec))


def test_null_arguments_return_invalid():
    lib = L.lib()
    assert lib.mfq_amd_dequant(None, 0, None, None) == L.ERR_INVALID
    assert lib.mfq_amd_topk(None, 0, 1, 8, 2, 1, 1e-20, 1.0, None, None, None) == L.ERR_INVALID
    assert lib.mfq_amd_grouped_matmul_workspace(4, 2, 8) > 0
    assert lib.mfq_amd_grouped_matmul_workspace(-1, 2, 8) == 0


# ------------------------------------------------------------------ hostile lengths ----
def _nint_header(out, ng, neuron_len, gs=24, bits=4, sub=6):
    import struct
    return struct.pack("<BBiiiI", bits | 0x80, sub, gs, 0, neuron_len, 2) + struct.pack("<qq", out, neuron_len) + \
        struct.pack("<II", out, ng)


def test_blobs_with_huge_counts_are_rejected_before_anything_is_allocated():
    """Header counts the remaining bytes cannot back must fail as a status code: a 40-byte NINT blob that names
    2^32 - 1 rows, an NVQ blob with 2^32 - 1 rows, an MXFP4 blob whose dimensions overflow the byte count."""
    import struct
    status, _ = _load("NINT", _nint_header(0xFFFFFFFF, 4, 96) + b"\0" * 8)
    assert status == L.ERR_INVALID, L.lib().mfq_amd_last_error()
    status, _ = _load("NINT", _nint_header(0xFFFFFFFF, 0xFFFFFFFF, 96) + b"\0" * 8)
    assert status == L.ERR_INVALID
    # rows x groups fits, but the code stream does not
    status, _ = _load("NINT", _nint_header(1 << 20, 4, 96) + b"\0" * (4 << 20) + b"\0" * 64)
    assert status == L.ERR_INVALID and b"truncated" in L.lib().mfq_amd_last_error()
    rng = np.random.default_rng(2)
    good = bytearray(nvq.pack_nvq(nvq_quant.random_nvq(4, 96, nvq.NVQ3_D4, rng)))
    rows_at = 20 + 16
    assert struct.unpack_from("<I", good, rows_at)[0] == 4
    struct.pack_into("<I", good, rows_at, 0xFFFFFFFF)
    struct.pack_into("<q", good, 20, 0xFFFFFFFF)
    status, _ = _load("NVQ", bytes(good))
    assert status == L.ERR_INVALID and b"truncated" in L.lib().mfq_amd_last_error()
    mxb = bytearray(mx.pack_mx(mx.random_mxfp4(2, 32, rng)))
    for rows, cols in ((1 << 62, 32), (1 << 40, 1 << 40), ((1 << 63) + 2, 32)):
        struct.pack_into("<6Q", mxb, 8, rows, cols, rows, cols // 2, rows, cols // 32)
        status, _ = _load("MXFP4", bytes(mxb))
        assert status == L.ERR_INVALID, (rows, cols)


@pytest.mark.parametrize("payload_len,runtime_len", [((1 << 63) - 1, 0), ((1 << 64) - 1, 0), (0, (1 << 63) - 8),
                                                     ((1 << 63) - 40, 64), (1 << 62, 1 << 62)])
def test_mfe_lengths_near_the_top_of_the_range_do_not_wrap(payload_len, runtime_len):
    """payload_len / runtime_len are unsigned 64-bit fields: a value near INT64_MAX must not pass the bounds check
    by overflowing offset + length (cpp_runtime/backends/cuda/ops/moe.cpp:70-87 compares against the bytes left)."""
    import struct
    rng = np.random.default_rng(4)
    payload = nint.pack_nint(nint_quant.random_codes(4, 48, nint.NintSpec(4, 24, 6), rng))
    head = struct.pack("<4sIIII", b"MFE1", 1, 4, 48, 1)
    blob = head + struct.pack("<IIQQ", 1, 4, payload_len, runtime_len) + np.asarray([0], "<i4").tobytes() + b"NINT" + payload
    status, _ = _mfe_status(blob)
    assert status == L.ERR_INVALID and b"truncated" in L.lib().mfq_amd_last_error()


def test_mfe_pool_with_more_experts_than_the_tensor_is_rejected():
    import struct
    blob = struct.pack("<4sIIII", b"MFE1", 2, 4, 48, 1) + struct.pack("<IIQQ", 0xFFFFFFF0, 4, 16, 0) + b"\0" * 64
    status, _ = _mfe_status(blob)
    assert status == L.ERR_INVALID


@pytest.mark.parametrize("cut", [1, 9, 40, 200])
@pytest.mark.parametrize("family", ["NVQ", "NVQJ", "MXFP4", "MFE"])
def test_truncated_blobs_of_every_family_are_rejected(family, cut):
    rng = np.random.default_rng(13)
    if family == "NVQ":
        blob, load = nvq.pack_nvq(nvq_quant.random_nvq(4, 96, nvq.NVQ3_D4, rng)), lambda b: _load("NVQ", b)[0]
    elif family == "NVQJ":
        blob, load = nvq.pack_nvq(nvq_quant.random_nvq_jsc(4, 96, nvq.NVQ3_D4_1024, rng)), lambda b: _load("NVQ", b)[0]
    elif family == "MXFP4":
        blob, load = mx.pack_mx(mx.random_mxfp4(4, 64, rng)), lambda b: _load("MXFP4", b)[0]
    else:
        pools = [MFE.MfePool(np.array([0, 1], dtype=np.int32), nint_quant.random_codes(8, 96, nint.NintSpec(4, 24, 6), rng))]
        blob, load = MFE.pack_mfe(MFE.MfeTensor((2, 4, 96), pools)), lambda b: _mfe_status(b)[0]
    assert load(blob) == 0
    assert load(blob[:-cut]) == L.ERR_INVALID
    assert load(blob[:min(cut, len(blob) - 1)]) == L.ERR_INVALID
    assert load(blob + b"\0") == L.ERR_INVALID


# --------------------------------------------------------------- descriptor checks ----
def _nint_view(rng, rows=8, width=96, bits=4, gs=24, out_per_expert=4):
    t = nint_quant.random_codes(rows, width, nint.NintSpec(bits, gs, 6), rng)
    status, handle = _load("NINT", nint.pack_nint(t), out_per_expert)
    assert status == 0
    view = L.Projection()
    assert L.lib().mfq_amd_tensor_host_view(handle, C.byref(view)) == 0
    return view, handle


def test_nint_descriptor_with_short_stream_or_stride_is_rejected():
    """The checks of the reference's validate() (cpp_runtime/backends/cpu/ops/packed_nint.cpp:15-34) a host can make
    without reading device memory: the last expert's rows fit the stream, an expert's rows fit its stride, and the
    code width is 0..8.  Validation runs before any device call, so this needs no GPU."""
    rng = np.random.default_rng(17)
    lib = L.lib()
    view, handle = _nint_view(rng)
    stream = 4 * view.groups * view.group_size * 4 // 8

    def status_of(v):
        return lib.mfq_amd_dequant(C.byref(v), 0, None, None)

    bad = L.Projection.from_buffer_copy(view); bad.sizes[0] = view.q_expert_stride + stream - 1
    assert status_of(bad) == L.ERR_INVALID and b"exceeds storage" in lib.mfq_amd_last_error()
    bad = L.Projection.from_buffer_copy(view); bad.q_expert_stride = stream - 1
    assert status_of(bad) == L.ERR_INVALID and b"stride" in lib.mfq_amd_last_error()
    bad = L.Projection.from_buffer_copy(view); bad.uniform_bits = 9
    assert status_of(bad) == L.ERR_INVALID and b"width" in lib.mfq_amd_last_error()
    bad = L.Projection.from_buffer_copy(view); bad.uniform_bits = 0; bad.sizes[0] = view.q_expert_stride + stream // 4 - 1
    assert status_of(bad) == L.ERR_INVALID                       # per-row widths: at least one bit per code
    ok = L.Projection.from_buffer_copy(view); ok.sizes[0] = view.q_expert_stride + stream
    assert status_of(ok) == L.ERR_INVALID and b"null" in lib.mfq_amd_last_error()   # passes validation; out is null
    lib.mfq_amd_tensor_free(handle)


def test_decode_token_limit_is_clamped_to_one_thread_per_pair():
    lib = L.lib()
    assert lib.mfq_amd_moe_ffn_decode_limit(0, 10) == 32
    assert lib.mfq_amd_moe_ffn_decode_limit(128, 10) == 102          # 1024 threads / 10 routes
    assert lib.mfq_amd_moe_ffn_decode_limit(128, 8) == 128
    assert lib.mfq_amd_moe_ffn_decode_limit(4096, 1) == 1024
    assert lib.mfq_amd_moe_ffn_decode_limit(64, 32) == 32
    assert lib.mfq_amd_moe_ffn_decode_limit(16, 0) == 0
    for top_k in range(1, 33):
        for requested in (0, 1, 31, 32, 33, 128, 1024, 100000):
            limit = lib.mfq_amd_moe_ffn_decode_limit(requested, top_k)
            assert 1 <= limit and limit * top_k <= 1024
