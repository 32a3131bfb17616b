"""ctypes doorway to the CPU oracle (oracle/liboracle.so) and, when built, to the
reference's own CPU library (oracle/_ref/libmfq_ref.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py -- never by the mfq_amd package.

Also holds a numpy restatement of the reference loaders that turn canonical tensors
into the runtime packed layout the kernels execute
(cpp_runtime/backends/cuda/ops/nint.cpp:750-964 unpack_nint, :1384-1459
to_device_mfe_nint; ops/vq.cpp:1030-1330 unpack_nvq), used to feed the oracle and to
cross-check the product's C++ loader.
"""

from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
_u8p, _i8p, _i32p, _i64p, _f32p, _u16p = (C.POINTER(t) for t in
                                          (C.c_uint8, C.c_int8, C.c_int32, C.c_int64, C.c_float, C.c_uint16))


def build(ref: bool = True) -> None:
    subprocess.run(["make", "-C", str(HERE), "oracle"], check=True, stdout=subprocess.DEVNULL)
    if ref:
        subprocess.run(["make", "-C", str(HERE), "ref"], check=True, stdout=subprocess.DEVNULL)


def _ptr(a: np.ndarray, typ):
    return a.ctypes.data_as(typ)


class _NintView(C.Structure):
    _fields_ = [("packed", _u8p), ("packed_bytes", C.c_int64), ("row_bits", _u8p),
                ("row_bit_offsets", _i64p), ("group_scale", _u8p), ("group_min", _u8p),
                ("row_scale", _f32p), ("row_min", _f32p),
                ("outputs", C.c_int64), ("width", C.c_int64), ("group_size", C.c_int64)]


class _NvqView(C.Structure):
    _fields_ = [("indices", _u8p), ("index_bytes", C.c_int64), ("aux", _u8p), ("aux_bytes", C.c_int64),
                ("states", _u8p), ("state_bytes", C.c_int64), ("anchors", _f32p), ("metadata", _i8p),
                ("format", C.c_int), ("state_bits", C.c_int), ("sign_mode", C.c_int),
                ("outputs", C.c_int64), ("width", C.c_int64), ("row_offset", C.c_int64)]


class _MxView(C.Structure):
    _fields_ = [("values", _u8p), ("scales", _u8p), ("outputs", C.c_int64), ("width", C.c_int64)]


class _Projection(C.Structure):
    _fields_ = [("family", C.c_int), ("nint", _NintView), ("nvq", _NvqView), ("mxfp4", _MxView)]


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        path = HERE / "liboracle.so"
        if not path.exists():
            build(ref=False)
        _lib = C.CDLL(str(path))
        L = _lib
        L.orc_bits_at.restype = C.c_uint32
        L.orc_bits_at.argtypes = [_u8p, C.c_int64, C.c_int64, C.c_int]
        L.orc_pack_bits.argtypes = [C.POINTER(C.c_uint32), C.c_int64, C.c_int, _u8p, C.c_int64]
        L.orc_f32_to_f16.restype = C.c_uint16; L.orc_f32_to_f16.argtypes = [C.c_float]
        L.orc_f64_to_f16.restype = C.c_uint16; L.orc_f64_to_f16.argtypes = [C.c_double]
        L.orc_f16_to_f32.restype = C.c_float; L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_f32_to_bf16.restype = C.c_uint16; L.orc_f32_to_bf16.argtypes = [C.c_float]
        L.orc_expf.restype = C.c_float; L.orc_expf.argtypes = [C.c_float]
        L.orc_swiglu_f16.restype = C.c_uint16; L.orc_swiglu_f16.argtypes = [C.c_uint16, C.c_uint16, C.c_float]
        L.orc_swiglu_array.argtypes = [_u16p, _u16p, C.c_int64, C.c_float, _u16p]
        L.orc_relu2_array.argtypes = [_u16p, C.c_int64, _u16p]
        L.orc_nint_validate.restype = C.c_int; L.orc_nint_validate.argtypes = [C.POINTER(_NintView)]
        L.orc_projection_dequant.argtypes = [C.POINTER(_Projection), _f32p]
        L.orc_projection_rows.argtypes = [C.POINTER(_Projection), C.c_int, _f32p, C.c_int64, C.c_int64,
                                          _f32p, C.c_int64, C.c_int64, C.c_int64]
        L.orc_nvq_decode_group.argtypes = [C.POINTER(_NvqView), C.c_int64, C.c_int, C.c_uint32, _i8p]
        L.orc_expert_ffn.argtypes = [C.POINTER(_Projection)] * 3 + [C.c_int, _f32p, C.c_int64, C.c_float,
                                                                     _f32p, _f32p, _f32p, _f32p]
        L.orc_topk.argtypes = [_f32p, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, _i32p, _f32p]
        L.orc_router_logits.argtypes = [_f32p, _f32p, C.c_int64, C.c_int, C.c_int64, _f32p]
        L.orc_route_plan.argtypes = [_i32p, C.c_int64, C.c_int, C.c_int, _i32p, _i32p, _i32p, _i32p, _i32p]
        L.orc_weighted_reduce.argtypes = [_u16p, _f32p, C.c_int64, C.c_int, C.c_int64, _f32p]
        L.orc_add_shared_gate.argtypes = [_u16p, _u16p, _f32p, C.c_int64, C.c_int64, _u16p]
        L.orc_weighted_reduce_shared_gate.argtypes = [_u16p, _f32p, _u16p, _f32p, C.c_int64, C.c_int, C.c_int64, _u16p]
    return _lib


def ref_lib():
    """The reference's CPU library, or None when oracle/_ref was never built."""
    global _ref
    if _ref is None:
        path = HERE / "_ref" / "libmfq_ref.so"
        if not path.exists():
            return None
        _ref = C.CDLL(str(path))
        R = _ref
        nint_args = [_u8p, C.c_int64, _u8p, _i64p, _u8p, _u8p, _f32p, _f32p, C.c_int64, C.c_int64, C.c_int64,
                     _f32p, C.c_int64, C.c_int64, _f32p, C.c_int64]
        R.ref_packed_nint_matmul.restype = C.c_int
        R.ref_packed_nint_matmul.argtypes = nint_args + [C.c_int, C.c_int]
        R.ref_packed_nint_rows.restype = None
        R.ref_packed_nint_rows.argtypes = nint_args + [C.c_int64, C.c_int64, C.c_int]
        R.ref_nvq_rows.restype = C.c_int
        R.ref_nvq_rows.argtypes = [C.c_int, _u8p, C.c_int64, _u8p, C.c_int64, _u8p, C.c_int64, C.c_int, _f32p,
                                   C.POINTER(_i8p), _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int64,
                                   _f32p, C.c_int64, C.c_int64, _f32p, C.c_int64, C.c_int64, C.c_int64, C.c_int]
        R.ref_scaled_i8_dot.restype = C.c_float
        R.ref_scaled_i8_dot.argtypes = [_i8p, _f32p, C.c_int, C.c_float, C.c_int]
        R.ref_has_avx2.restype = C.c_int
        R.ref_pool_participants.restype = C.c_int
        if hasattr(R, "ref_layer"):
            R.ref_layer.restype = C.c_int
            R.ref_layer.argtypes = [C.POINTER(_Projection), _i32p, _i32p, C.c_int, _f32p, C.c_int64, C.c_int64, C.c_int,
                                    C.POINTER(_LayerFns), _f32p]
    return _ref


class _LayerFns(C.Structure):
    """``ref_layer_fns`` of ref_shim.cpp: the pieces of a layer the reference's CPU library does not hold."""
    _fields_ = [("mx_rows", C.c_void_p), ("swiglu", C.c_void_p), ("f32_to_f16", C.c_void_p), ("f16_to_f32", C.c_void_p),
                ("nvq_multiplier", C.c_void_p), ("nvq_bank", C.c_void_p)]


class RefLayer:
    """One routed MoE layer prepared for ref_layer(): a single C call runs every routed expert of the batch through
    the reference's CPU rows kernels (NINT, NVQ) and the C restatement (MXFP4 rows, SwiGLU chain)."""

    def __init__(self, layouts_by_expert: dict, tokens_by_expert: dict, x: np.ndarray):
        experts = sorted(tokens_by_expert)
        self._keep = [tuple(Projection(L) for L in layouts_by_expert[e]) for e in experts]
        self.projections = (_Projection * (3 * len(experts)))()
        for i, triple in enumerate(self._keep):
            for j, proj in enumerate(triple):
                self.projections[3 * i + j] = proj.struct
        counts = [len(tokens_by_expert[e]) for e in experts]
        self.offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
        self.token_ids = np.concatenate([np.asarray(tokens_by_expert[e], dtype=np.int32) for e in experts]).astype(np.int32)
        self.x = np.ascontiguousarray(x, dtype=np.float32)
        self.hidden = int(self.x.shape[1])
        self.inter = int(self._keep[0][0].outputs)
        self.experts = len(experts)
        self.out = np.zeros((int(self.offsets[-1]), self.hidden), dtype=np.float32)
        L = lib()
        self.fns = _LayerFns(*[C.cast(getattr(L, name), C.c_void_p).value for name in
                               ("orc_mxfp4_rows", "orc_swiglu_array", "orc_f32_to_f16", "orc_f16_to_f32",
                                "orc_nvq_multiplier", "orc_nvq_bank")])

    def run(self, pooled: bool) -> np.ndarray:
        status = ref_lib().ref_layer(self.projections, _ptr(self.offsets, _i32p), _ptr(self.token_ids, _i32p), self.experts,
                                     _ptr(self.x, _f32p), self.hidden, self.inter, int(pooled), C.byref(self.fns),
                                     _ptr(self.out, _f32p))
        if status:
            raise RuntimeError("the reference has no fused rows kernel for one of the formats on this host")
        return self.out


# ------------------------------------------------------------------------------
# runtime packed layout (numpy restatement of the reference loaders)
# ------------------------------------------------------------------------------

def _bitstream(values: np.ndarray, bits: int) -> np.ndarray:
    flat = np.ascontiguousarray(values).reshape(-1).astype(np.uint32)
    planes = ((flat[:, None] >> np.arange(bits, dtype=np.uint32)[None, :]) & 1).astype(np.uint8)
    return np.packbits(planes.reshape(-1), bitorder="little")


def nint_runtime(t, out_per_expert: int | None = None) -> dict:
    """Runtime NINT layout.  ``out_per_expert=None``: dense tensor layout of unpack_nint
    (q cohorts in ascending q width, then 8 zero guard bytes; nint.cpp:881-935).  Otherwise the
    MFE layout of to_device_mfe_nint (per expert a stream of ``ceil(max_bits/8)+8`` bytes with
    rows bit-contiguous in row order and expert-relative offsets; nint.cpp:1384-1438)."""
    out, ng, gs = t.q.shape
    bits = np.asarray(t.row_q_bits, dtype=np.int64)
    row_payload = ng * gs * bits
    if out_per_expert is None:
        chunks, offsets, cursor = [], np.zeros(out, dtype=np.int64), 0
        for width in range(1, 9):
            rows = np.flatnonzero(bits == width)
            if not rows.size:
                continue
            stream = _bitstream(t.q[rows], width)
            offsets[rows] = cursor * 8 + np.arange(rows.size, dtype=np.int64) * ng * gs * width
            chunks.append(stream)
            cursor += stream.size
        packed = np.concatenate(chunks + [np.zeros(8, dtype=np.uint8)])
        stride = 0
    else:
        experts = out // out_per_expert
        per_expert_bits = row_payload.reshape(experts, out_per_expert).sum(-1)
        stride = int((per_expert_bits.max() + 7) // 8 + 8)
        packed = np.zeros(experts * stride, dtype=np.uint8)
        offsets = np.zeros(out, dtype=np.int64)
        for e in range(experts):
            rows = slice(e * out_per_expert, (e + 1) * out_per_expert)
            rel = np.concatenate([[0], np.cumsum(row_payload[rows])[:-1]])
            offsets[rows] = rel
            if np.all(bits[rows] == bits[rows][0]):
                stream = _bitstream(t.q[rows], int(bits[rows][0]))
            else:
                pieces = [np.unpackbits(_bitstream(t.q[r], int(bits[r])), bitorder="little")[: row_payload[r]]
                          for r in range(rows.start, rows.stop)]
                stream = np.packbits(np.concatenate(pieces), bitorder="little")
            packed[e * stride : e * stride + stream.size] = stream
    return dict(family=1, packed=packed, row_bits=np.ascontiguousarray(t.row_q_bits, dtype=np.uint8),
                row_bit_offsets=offsets, group_scale=np.ascontiguousarray(t.sub_scale, dtype=np.uint8).reshape(-1),
                group_min=np.ascontiguousarray(t.sub_min, dtype=np.uint8).reshape(-1),
                row_scale=np.ascontiguousarray(t.neuron_scale, dtype=np.float32),
                row_min=np.ascontiguousarray(t.neuron_min, dtype=np.float32),
                outputs=out, width=t.neuron_len, group_size=gs, groups=ng, q_expert_stride=stride)


def nvq_runtime(t) -> dict:
    """Runtime NVQ layout: the blob's three bit streams verbatim, anchors as fp32 and the
    codebook metadata (plain: expanded ``[entries][dim]`` int8 table; JSC: 64-byte header +
    banks) -- ops/vq.cpp:1278-1330."""
    from mfq_amd.formats import nvq as F
    spec = t.spec
    jsc = isinstance(t, F.NvqJscTensor)
    if jsc:
        metadata = np.frombuffer(F.pack_jsc_tables(t.scale_lut, t.bank_for_state, t.codebooks), dtype=np.int8).copy()
        states = t.state
    else:
        table = F.codebook_for(spec) if t.codebook is None else t.codebook
        metadata = np.ascontiguousarray(table, dtype=np.int8).reshape(-1).copy()
        states = t.sub_scale
    return dict(family=2, indices=_bitstream(t.indices, spec.index_bits), aux=_bitstream(t.signs, 7),
                states=_bitstream(states, spec.sub_bits),
                anchors=np.ascontiguousarray(t.neuron_scale, dtype=np.float32), metadata=metadata,
                format=t.runtime_format, state_bits=spec.sub_bits,
                sign_mode=1 if spec.sign_mode == "index_parity" else 0,
                outputs=int(np.asarray(t.neuron_scale).size), width=t.neuron_len)


def mxfp4_runtime(t) -> dict:
    return dict(family=3, values=np.ascontiguousarray(t.values, dtype=np.uint8).reshape(-1),
                scales=np.ascontiguousarray(t.scales, dtype=np.uint8).reshape(-1),
                outputs=t.shape[0], width=t.shape[1])


def runtime_layout(t, out_per_expert: int | None = None) -> dict:
    from mfq_amd.formats.mx import Mxfp4Tensor
    from mfq_amd.formats.nint import NintTensor
    if isinstance(t, NintTensor):
        return nint_runtime(t, out_per_expert)
    if isinstance(t, Mxfp4Tensor):
        return mxfp4_runtime(t)
    return nvq_runtime(t)


def slice_rows(layout: dict, begin: int, end: int) -> dict:
    """View of rows [begin, end) of a runtime layout (one expert of a pool)."""
    L = dict(layout)
    n = end - begin
    if L["family"] == 1:
        g = L["groups"]
        stride = L["q_expert_stride"]
        if stride:
            per_expert = n
            e = begin // per_expert
            L["packed"] = L["packed"][e * stride : (e + 1) * stride]
        for key in ("row_bits", "row_bit_offsets", "row_scale", "row_min"):
            L[key] = L[key][begin:end]
        for key in ("group_scale", "group_min"):
            L[key] = L[key][begin * g : end * g]
    elif L["family"] == 2:
        L["row_offset"] = L.get("row_offset", 0) + begin      # streams and anchors stay whole-pool
    else:
        w = L["width"]
        L["values"] = L["values"][begin * (w // 2) : end * (w // 2)]
        L["scales"] = L["scales"][begin * (w // 32) : end * (w // 32)]
    L["outputs"] = n
    return L


class Projection:
    """Owns the numpy arrays of one runtime layout and the C struct that points at them."""

    def __init__(self, layout: dict):
        self.layout = layout
        self.struct = _Projection()
        self.struct.family = layout["family"]
        L = layout
        if L["family"] == 1:
            v = self.struct.nint
            v.packed, v.packed_bytes = _ptr(L["packed"], _u8p), L["packed"].size
            v.row_bits = _ptr(L["row_bits"], _u8p)
            v.row_bit_offsets = _ptr(L["row_bit_offsets"], _i64p)
            v.group_scale, v.group_min = _ptr(L["group_scale"], _u8p), _ptr(L["group_min"], _u8p)
            v.row_scale, v.row_min = _ptr(L["row_scale"], _f32p), _ptr(L["row_min"], _f32p)
            v.outputs, v.width, v.group_size = L["outputs"], L["width"], L["group_size"]
        elif L["family"] == 2:
            v = self.struct.nvq
            v.indices, v.index_bytes = _ptr(L["indices"], _u8p), L["indices"].size
            v.aux, v.aux_bytes = _ptr(L["aux"], _u8p), L["aux"].size
            v.states, v.state_bytes = _ptr(L["states"], _u8p), L["states"].size
            v.anchors, v.metadata = _ptr(L["anchors"], _f32p), _ptr(L["metadata"], _i8p)
            v.format, v.state_bits, v.sign_mode = L["format"], L["state_bits"], L["sign_mode"]
            v.outputs, v.width = L["outputs"], L["width"]
            v.row_offset = L.get("row_offset", 0)
        else:
            v = self.struct.mxfp4
            v.values, v.scales = _ptr(L["values"], _u8p), _ptr(L["scales"], _u8p)
            v.outputs, v.width = L["outputs"], L["width"]

    @property
    def outputs(self) -> int:
        return int(self.layout["outputs"])

    @property
    def width(self) -> int:
        return int(self.layout["width"])

    def dequant(self) -> np.ndarray:
        out = np.empty((self.outputs, self.width), dtype=np.float32)
        lib().orc_projection_dequant(C.byref(self.struct), _ptr(out, _f32p))
        return out

    def rows(self, x: np.ndarray, order: int = 0, begin: int = 0, end: int | None = None) -> np.ndarray:
        """y[b, r] for rows [begin, end); other columns of the result are zero."""
        x = np.ascontiguousarray(x, dtype=np.float32)
        batch = x.shape[0]
        y = np.zeros((batch, self.outputs), dtype=np.float32)
        end = self.outputs if end is None else end
        lib().orc_projection_rows(C.byref(self.struct), order, _ptr(x, _f32p), batch, x.shape[1],
                                  _ptr(y, _f32p), self.outputs, begin, end)
        return y


def relu2_array(up_f16: np.ndarray) -> np.ndarray:
    """half(relu(up)^2), the gate-less expert activation (mfq/kernels/cuda/mfe_ffn.h:107-110)."""
    u = np.ascontiguousarray(up_f16, dtype=np.float16)
    out = np.empty_like(u)
    lib().orc_relu2_array(_ptr(u.view(np.uint16), _u16p), u.size, _ptr(out.view(np.uint16), _u16p))
    return out


def expert_ffn(gate: Projection, up: Projection, down: Projection, x: np.ndarray, order: int = 0,
               swiglu_limit: float = 0.0, activation: int = 0) -> np.ndarray:
    """activation 1: hidden = half(relu(half(up . x))^2), no gate projection (``gate`` is ignored)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    if activation == 1:
        hidden = relu2_array(up.rows(x, order).astype(np.float16)).astype(np.float32)
        return down.rows(hidden, order)
    count, inter = x.shape[0], gate.outputs
    g = np.empty((count, inter), dtype=np.float32)
    u = np.empty_like(g)
    h = np.empty_like(g)
    out = np.empty((count, down.outputs), dtype=np.float32)
    lib().orc_expert_ffn(C.byref(gate.struct), C.byref(up.struct), C.byref(down.struct), order,
                         _ptr(x, _f32p), count, swiglu_limit, _ptr(g, _f32p), _ptr(u, _f32p),
                         _ptr(h, _f32p), _ptr(out, _f32p))
    return out


def topk(logits: np.ndarray, k: int, normalize: bool = True, floor: float = 1e-20, scale: float = 1.0):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    tokens, experts = logits.shape
    ids = np.empty((tokens, k), dtype=np.int32)
    weights = np.empty((tokens, k), dtype=np.float32)
    lib().orc_topk(_ptr(logits, _f32p), tokens, experts, k, int(normalize), floor, scale,
                   _ptr(ids, _i32p), _ptr(weights, _f32p))
    return ids, weights


def router_logits(x: np.ndarray, router: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    router = np.ascontiguousarray(router, dtype=np.float32)
    logits = np.empty((x.shape[0], router.shape[0]), dtype=np.float32)
    lib().orc_router_logits(_ptr(x, _f32p), _ptr(router, _f32p), x.shape[0], router.shape[0], x.shape[1],
                            _ptr(logits, _f32p))
    return logits


def route_plan(ids: np.ndarray, experts: int, tile_m: int = 8):
    flat = np.ascontiguousarray(ids, dtype=np.int32).reshape(-1)
    counts = np.zeros(experts, dtype=np.int32)
    bounds = np.zeros(experts + 1, dtype=np.int32)
    tile_bounds = np.zeros(experts + 1, dtype=np.int32)
    tile_experts = np.zeros(flat.size + experts, dtype=np.int32)
    ids_dst = np.zeros(flat.size, dtype=np.int32)
    lib().orc_route_plan(_ptr(flat, _i32p), flat.size, experts, tile_m, _ptr(counts, _i32p), _ptr(bounds, _i32p),
                         _ptr(tile_bounds, _i32p), _ptr(tile_experts, _i32p), _ptr(ids_dst, _i32p))
    return dict(counts=counts, expert_bounds=bounds, tile_bounds=tile_bounds,
                tile_experts=tile_experts[: tile_bounds[-1]], ids_dst=ids_dst[: bounds[-1]])


def f32_to_f16_bits(x: np.ndarray) -> np.ndarray:
    f = np.vectorize(lambda v: lib().orc_f32_to_f16(float(v)), otypes=[np.uint16])
    return f(np.asarray(x, dtype=np.float32))


def swiglu_array(gate_f16: np.ndarray, up_f16: np.ndarray, swiglu_limit: float = 0.0) -> np.ndarray:
    g = np.ascontiguousarray(gate_f16, dtype=np.float16)
    u = np.ascontiguousarray(up_f16, dtype=np.float16)
    out = np.empty(g.shape, dtype=np.float16)
    lib().orc_swiglu_array(_ptr(g.view(np.uint16), _u16p), _ptr(u.view(np.uint16), _u16p), g.size, swiglu_limit,
                           _ptr(out.view(np.uint16), _u16p))
    return out


def weighted_reduce(pairs_f16: np.ndarray, weights: np.ndarray) -> np.ndarray:
    tokens, routes, width = pairs_f16.shape
    pairs = np.ascontiguousarray(pairs_f16.view(np.uint16))
    weights = np.ascontiguousarray(weights, dtype=np.float32)
    out = np.empty((tokens, width), dtype=np.float32)
    lib().orc_weighted_reduce(_ptr(pairs, _u16p), _ptr(weights, _f32p), tokens, routes, width, _ptr(out, _f32p))
    return out


def add_shared_gate(routed_f16: np.ndarray, shared_f16: np.ndarray, gate_logits: np.ndarray) -> np.ndarray:
    """half(routed + sigmoid(gate_logits[row]) * shared), mfq/kernels/cuda/moe.cu:1557-1571."""
    rows, width = routed_f16.shape
    routed = np.ascontiguousarray(routed_f16, dtype=np.float16)
    shared = np.ascontiguousarray(shared_f16, dtype=np.float16)
    gate = np.ascontiguousarray(gate_logits, dtype=np.float32)
    out = np.empty((rows, width), dtype=np.float16)
    lib().orc_add_shared_gate(_ptr(routed.view(np.uint16), _u16p), _ptr(shared.view(np.uint16), _u16p), _ptr(gate, _f32p),
                              rows, width, _ptr(out.view(np.uint16), _u16p))
    return out


def weighted_reduce_shared_gate(pairs_f16: np.ndarray, weights: np.ndarray, shared_f16: np.ndarray,
                                gate_logits: np.ndarray) -> np.ndarray:
    """half(half(sum_r w * pair) + sigmoid(gate_logits[token]) * shared), mfq/kernels/cuda/moe.cu:1573-1596."""
    tokens, routes, width = pairs_f16.shape
    pairs = np.ascontiguousarray(pairs_f16, dtype=np.float16)
    shared = np.ascontiguousarray(shared_f16, dtype=np.float16)
    weights = np.ascontiguousarray(weights, dtype=np.float32)
    gate = np.ascontiguousarray(gate_logits, dtype=np.float32)
    out = np.empty((tokens, width), dtype=np.float16)
    lib().orc_weighted_reduce_shared_gate(_ptr(pairs.view(np.uint16), _u16p), _ptr(weights, _f32p),
                                          _ptr(shared.view(np.uint16), _u16p), _ptr(gate, _f32p), tokens, routes, width,
                                          _ptr(out.view(np.uint16), _u16p))
    return out


def shared_expert_epilogue(routed_sum_f32: np.ndarray, shared_f16: np.ndarray, gate: np.ndarray) -> np.ndarray:
    """The last lines of mfe_ffn_down_reduce_kernel (mfq/kernels/cuda/mfe_ffn_device.cuh:1249-1263): the route-ordered fp32
    sum is rounded to fp16, the shared expert's fp16 output is multiplied with the token's evaluated gate value in fp32
    (and the product rounded to fp16 when the gate values are fp16: shared_product_half), and the two are added in fp32.
    ``gate``: [tokens] float32, float16 or bfloat16-as-float32 values."""
    routed = np.asarray(routed_sum_f32, dtype=np.float32).astype(np.float16).astype(np.float32)
    product_half = np.asarray(gate).dtype == np.float16
    g = np.asarray(gate).astype(np.float32)[:, None]
    contribution = np.asarray(shared_f16, dtype=np.float16).astype(np.float32) * g
    if product_half:
        contribution = contribution.astype(np.float16).astype(np.float32)
    return (routed + contribution).astype(np.float32)


def moe_layer(x: np.ndarray, ids: np.ndarray, weights: np.ndarray, expert_projections, order: int = 0,
              swiglu_limit: float = 0.0, activation: int = 0) -> np.ndarray:
    """Whole MoE FFN on the CPU: per routed pair the expert FFN of
    cuda/storage/moe_ffn_pipeline.cpp:142-180, pair outputs rounded to fp16
    (moe_ffn_pipeline.cpp:187 workspace type), then the route-ordered fp32 reduce.
    ``expert_projections(e)`` returns (gate, up, down) :class:`Projection` of expert ``e``."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    tokens, routes = ids.shape
    width = x.shape[1]
    pairs = np.zeros((tokens, routes, width), dtype=np.float16)
    by_expert: dict[int, list[tuple[int, int]]] = {}
    for t in range(tokens):
        for r in range(routes):
            by_expert.setdefault(int(ids[t, r]), []).append((t, r))
    for e, slots in by_expert.items():
        gate, up, down = expert_projections(e)
        rows = np.stack([x[t] for t, _ in slots])
        y = expert_ffn(gate, up, down, rows, order, swiglu_limit, activation)
        for (t, r), row in zip(slots, y):
            pairs[t, r] = row.astype(np.float16)
    return weighted_reduce(pairs, weights)


# ------------------------------------------------------------------------------
# the reference's own CPU kernels
# ------------------------------------------------------------------------------

def ref_nint_matmul(layout: dict, x: np.ndarray, threads: int = 1, scalar: bool = False) -> np.ndarray:
    R = ref_lib()
    x = np.ascontiguousarray(x, dtype=np.float32)
    L = layout
    y = np.zeros((x.shape[0], L["outputs"]), dtype=np.float32)
    status = R.ref_packed_nint_matmul(
        _ptr(L["packed"], _u8p), L["packed"].size, _ptr(L["row_bits"], _u8p), _ptr(L["row_bit_offsets"], _i64p),
        _ptr(L["group_scale"], _u8p), _ptr(L["group_min"], _u8p), _ptr(L["row_scale"], _f32p),
        _ptr(L["row_min"], _f32p), L["outputs"], L["width"], L["group_size"],
        _ptr(x, _f32p), x.shape[0], x.shape[1], _ptr(y, _f32p), L["outputs"], threads, int(scalar))
    if status:
        raise ValueError("reference rejected the packed NINT descriptor")
    return y


def ref_nint_rows_pooled(layout: dict, x: np.ndarray, pooled: bool = True) -> np.ndarray:
    """Rows kernel the reference selects per expert job, split over its pinned expert pool."""
    R = ref_lib()
    x = np.ascontiguousarray(x, dtype=np.float32)
    L = layout
    y = np.zeros((x.shape[0], L["outputs"]), dtype=np.float32)
    R.ref_packed_nint_rows(
        _ptr(L["packed"], _u8p), L["packed"].size, _ptr(L["row_bits"], _u8p), _ptr(L["row_bit_offsets"], _i64p),
        _ptr(L["group_scale"], _u8p), _ptr(L["group_min"], _u8p), _ptr(L["row_scale"], _f32p),
        _ptr(L["row_min"], _f32p), L["outputs"], L["width"], L["group_size"],
        _ptr(x, _f32p), x.shape[0], x.shape[1], _ptr(y, _f32p), L["outputs"], 0, L["outputs"], int(pooled))
    return y


def ref_nvq_rows(layout: dict, x: np.ndarray, pooled: bool = False) -> np.ndarray | None:
    """Rows [row_offset, row_offset + outputs) of the pool through nvq_rows_dot_kernel(format)."""
    R = ref_lib()
    x = np.ascontiguousarray(x, dtype=np.float32)
    L = layout
    proj = Projection(L)
    view = proj.struct.nvq
    nstates = 1 << L["state_bits"]
    banks = (_i8p * 16)()
    mult = np.zeros(16, dtype=np.float32)
    lib().orc_nvq_bank.restype = _i8p
    lib().orc_nvq_bank.argtypes = [C.POINTER(_NvqView), C.c_uint32]
    lib().orc_nvq_multiplier.restype = C.c_float
    lib().orc_nvq_multiplier.argtypes = [C.POINTER(_NvqView), C.c_uint32]
    for s in range(min(nstates, 16)):
        banks[s] = lib().orc_nvq_bank(C.byref(view), s)
        mult[s] = lib().orc_nvq_multiplier(C.byref(view), s)
    d4 = L["format"] in (3, 10, 11, 12, 15)
    width = L["width"]
    nvec = (width + (3 if d4 else 7)) // (4 if d4 else 8)
    first = int(L.get("row_offset", 0))
    total = int(L["anchors"].size)
    y = np.zeros((x.shape[0], total), dtype=np.float32)
    status = R.ref_nvq_rows(L["format"], _ptr(L["indices"], _u8p), L["indices"].size, _ptr(L["aux"], _u8p),
                            L["aux"].size, _ptr(L["states"], _u8p), L["states"].size, L["state_bits"],
                            _ptr(L["anchors"], _f32p), banks, _ptr(mult, _f32p), nvec, (width + 7) // 8,
                            (width + 23) // 24, L["sign_mode"], width, _ptr(x, _f32p), x.shape[0], x.shape[1],
                            _ptr(y, _f32p), total, first, first + L["outputs"], int(pooled))
    return None if status else np.ascontiguousarray(y[:, first:first + L["outputs"]])
