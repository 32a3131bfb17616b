"""Host-side mirror of the reference's operator interface for the MoE expert-FFN path,
on top of the C ABI.  torch supplies device memory and the current stream only; every
computation happens in libmfq_amd.so.

Reference counterparts (cpp_runtime/backends/cuda/ops/):
  PackedTensor          NintWeight / NvqWeight / Mxfp4Weight    include/nint.h:28-72, vq.h:16-55, mx.h:16-21
  dequantize            nint_decode_f32_cuda & friends          include/mfq_cuda_quant_ops.h:97-102
  matmul                nint_matmul / nvq_matmul / mxfp4_matmul include/nint.h:74-77, vq.h:71-74, mx.h:41-42
  moe_topk              moe_topk_cuda                           mfq/kernels/cuda/moe.cu:1953
  build_moe_route_plan  build_moe_route_plan                    moe.cpp:257-320
  MixedMoeRuntime       MixedMoeRuntime                         include/moe.h:133-189
  MfeFfnRuntime         MfeFfnRuntime                           include/mfe_ffn_runtime.h:9-97
"""

from __future__ import annotations

import ctypes as C

import numpy as np
import torch

from . import _lib as L
from .formats.mfe import MfeTensor, pack_mfe
from .formats.mx import Mxfp4Tensor, pack_mx
from .formats.nint import NintTensor, pack_nint
from .formats.nvq import pack_nvq

_DTYPES = {torch.float32: L.F32, torch.float16: L.F16, torch.bfloat16: L.BF16}


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported activation dtype {t.dtype}") from None


def pack_payload(tensor) -> tuple[str, bytes]:
    """(container dtype tag, canonical blob) of a format tensor."""
    if isinstance(tensor, NintTensor):
        return "NINT", pack_nint(tensor)
    if isinstance(tensor, Mxfp4Tensor):
        return "MXFP4", pack_mx(tensor)
    return "NVQ", pack_nvq(tensor)


class PackedTensor:
    """One packed weight tensor in the runtime layout (a dense matrix, or one MFE pool)."""

    def __init__(self, dtype: str, blob: bytes, out_per_expert: int = 0):
        handle = C.c_void_p()
        buf = (C.c_uint8 * len(blob)).from_buffer_copy(blob)
        L.check(L.lib().mfq_amd_tensor_load(dtype.encode(), buf, len(blob), out_per_expert, C.byref(handle)))
        self._handle = handle
        self.view = None

    @classmethod
    def from_tensor(cls, tensor, out_per_expert: int = 0) -> "PackedTensor":
        dtype, blob = pack_payload(tensor)
        return cls(dtype, blob, out_per_expert)

    def host_view(self) -> L.Projection:
        view = L.Projection()
        L.check(L.lib().mfq_amd_tensor_host_view(self._handle, C.byref(view)))
        return view

    def host_field(self, index: int, dtype, count: int) -> np.ndarray:
        view = self.host_view()
        size = count * np.dtype(dtype).itemsize
        raw = C.string_at(view.fields[index], size)
        return np.frombuffer(raw, dtype=dtype).copy()

    def cuda(self, expert_local: np.ndarray | None = None) -> "PackedTensor":
        view = L.Projection()
        if expert_local is None:
            L.check(L.lib().mfq_amd_tensor_upload(self._handle, None, 0, C.byref(view)))
        else:
            local = np.ascontiguousarray(expert_local, dtype=np.int32)
            L.check(L.lib().mfq_amd_tensor_upload(self._handle, local.ctypes.data, local.size, C.byref(view)))
        self.view = view
        return self

    def __del__(self):
        handle, self._handle = getattr(self, "_handle", None), None
        if handle and L is not None and getattr(L, "_lib", None) is not None:
            L._lib.mfq_amd_tensor_free(handle)


def dequantize(weight: PackedTensor, local_expert: int = 0) -> torch.Tensor:
    """Dense fp32 ``[output_rows, input_width]`` of one expert, bit-exact."""
    v = weight.view
    out = torch.empty((v.output_rows, v.input_width), dtype=torch.float32, device="cuda")
    L.check(L.lib().mfq_amd_dequant(C.byref(v), local_expert, out.data_ptr(), _stream()))
    return out


def matmul(weight: PackedTensor, x: torch.Tensor, local_expert: int = 0) -> torch.Tensor:
    """``x[B, K] -> y[B, N]`` fp32 (the nint_matmul / nvq_matmul / mxfp4_matmul entry)."""
    v = weight.view
    if x.dim() != 2 or not x.is_cuda:
        raise ValueError("x must be a CUDA [batch, width] tensor")
    x = x.contiguous()
    y = torch.empty((x.shape[0], v.output_rows), dtype=torch.float32, device="cuda")
    L.check(L.lib().mfq_amd_gemv(C.byref(v), local_expert, x.data_ptr(), _dtype_code(x), x.shape[0], x.stride(0),
                                 y.data_ptr(), y.stride(0), _stream()))
    return y


def router_logits(x: torch.Tensor, router: torch.Tensor) -> torch.Tensor:
    x, router = x.contiguous(), router.contiguous()
    logits = torch.empty((x.shape[0], router.shape[0]), dtype=torch.float32, device="cuda")
    L.check(L.lib().mfq_amd_router_logits(x.data_ptr(), _dtype_code(x), router.data_ptr(), _dtype_code(router),
                                          x.shape[0], router.shape[0], x.shape[1], logits.data_ptr(), _stream()))
    return logits


def moe_topk(logits: torch.Tensor, top_k: int, normalize: bool = True, norm_floor: float = 1e-20,
             scale: float = 1.0) -> tuple[torch.Tensor, torch.Tensor]:
    logits = logits.contiguous()
    tokens, experts = logits.shape
    ids = torch.empty((tokens, top_k), dtype=torch.int32, device="cuda")
    weights = torch.empty((tokens, top_k), dtype=torch.float32, device="cuda")
    L.check(L.lib().mfq_amd_topk(logits.data_ptr(), _dtype_code(logits), tokens, experts, top_k, int(normalize),
                                 norm_floor, scale, ids.data_ptr(), weights.data_ptr(), _stream()))
    return ids, weights


def moe_topk_into(logits: torch.Tensor, top_k: int, ids: torch.Tensor, weights: torch.Tensor, normalize: bool = True,
                  norm_floor: float = 1e-20, scale: float = 1.0) -> None:
    """moe_topk into caller-owned buffers (no allocation; usable under graph capture)."""
    tokens, experts = logits.shape
    L.check(L.lib().mfq_amd_topk(logits.data_ptr(), _dtype_code(logits), tokens, experts, top_k, int(normalize),
                                 norm_floor, scale, ids.data_ptr(), weights.data_ptr(), _stream()))


def build_moe_route_plan(ids: torch.Tensor, n_experts: int, tile_m: int = 8) -> dict:
    ids = ids.contiguous()
    tokens, k = ids.shape
    pairs = tokens * k
    i32 = dict(dtype=torch.int32, device="cuda")
    plan = dict(counts=torch.zeros(n_experts, **i32), expert_bounds=torch.zeros(n_experts + 1, **i32),
                tile_bounds=torch.zeros(n_experts + 1, **i32),
                tile_experts=torch.zeros(pairs // tile_m + n_experts + 1, **i32),
                ids_dst=torch.zeros(max(pairs, 1), **i32))
    L.check(L.lib().mfq_amd_route_plan(ids.data_ptr(), tokens, k, n_experts, tile_m, plan["counts"].data_ptr(),
                                       plan["expert_bounds"].data_ptr(), plan["tile_bounds"].data_ptr(),
                                       plan["tile_experts"].data_ptr(), plan["ids_dst"].data_ptr(), _stream()))
    return plan


class MixedMoeRuntime:
    """One logical ``[experts, out, in]`` tensor stored as per-format pools."""

    def __init__(self, mfe: MfeTensor):
        self.experts, self.out_per_expert, self.neuron_len = mfe.shape
        self.pools = []
        for pool in mfe.pools:
            local = np.full(self.experts, -1, dtype=np.int32)
            local[np.asarray(pool.expert_ids)] = np.arange(len(pool.expert_ids), dtype=np.int32)
            self.pools.append(PackedTensor.from_tensor(pool.tensor, self.out_per_expert).cuda(local))
        self._views = (L.Projection * len(self.pools))(*[p.view for p in self.pools])
        self.struct = L.MoeTensor(self._views, len(self.pools), self.experts, self.out_per_expert, self.neuron_len)

    @classmethod
    def from_dense(cls, tensor) -> "MixedMoeRuntime":
        """A single dense matrix as a one-expert tensor (no expert map): how a shared expert is handed to the FFN."""
        self = cls.__new__(cls)
        packed = PackedTensor.from_tensor(tensor, 0).cuda()
        self.experts, self.out_per_expert, self.neuron_len = 1, packed.view.output_rows, packed.view.input_width
        self.pools = [packed]
        self._views = (L.Projection * 1)(packed.view)
        self.struct = L.MoeTensor(self._views, 1, 1, self.out_per_expert, self.neuron_len)
        return self

    @classmethod
    def from_blob(cls, blob: bytes) -> "MixedMoeRuntime":
        """Through the C++ MFE container reader instead of the Python object model."""
        self = cls.__new__(cls)
        handle = C.c_void_p()
        buf = (C.c_uint8 * len(blob)).from_buffer_copy(blob)
        L.check(L.lib().mfq_amd_mfe_load(buf, len(blob), C.byref(handle)))
        info = [C.c_int32() for _ in range(4)]
        L.check(L.lib().mfq_amd_mfe_info(handle, *[C.byref(i) for i in info]))
        self.experts, self.out_per_expert, self.neuron_len = (i.value for i in info[:3])
        self._views = (L.Projection * info[3].value)()
        L.check(L.lib().mfq_amd_mfe_upload(handle, self._views, info[3].value))
        self._mfe_handle = handle
        self.pools = []
        self.struct = L.MoeTensor(self._views, info[3].value, self.experts, self.out_per_expert, self.neuron_len)
        return self

    def forward(self, x: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
        """``x[T, K]`` or ``x[T, k, K]`` -> fp16 ``[T, k, N]`` (MixedMoeRuntime::forward)."""
        x, ids = x.contiguous(), ids.contiguous()
        tokens, k = ids.shape
        rows_per_token = 1 if x.dim() == 2 else k
        out = torch.zeros((tokens, k, self.out_per_expert), dtype=torch.float16, device="cuda")
        nbytes = L.lib().mfq_amd_grouped_matmul_workspace(tokens, k, self.experts)
        workspace = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        L.check(L.lib().mfq_amd_grouped_matmul(C.byref(self.struct), x.data_ptr(), _dtype_code(x), rows_per_token,
                                               ids.data_ptr(), tokens, k, out.data_ptr(), workspace.data_ptr(),
                                               nbytes, _stream()))
        return out

    def __del__(self):
        handle = getattr(self, "_mfe_handle", None)
        if handle and L is not None and getattr(L, "_lib", None) is not None:
            self._mfe_handle = None
            L._lib.mfq_amd_mfe_free(handle)


class MfeFfnRuntime:
    """Routed expert FFN: gate/up -> SwiGLU -> down -> route-weighted reduce."""

    def __init__(self, gate: MixedMoeRuntime | None, up: MixedMoeRuntime, down: MixedMoeRuntime, top_k: int,
                 max_tokens: int, x_dtype: torch.dtype = torch.bfloat16, out_dtype: torch.dtype = torch.float32,
                 swiglu_limit: float = 0.0, decode_token_limit: int = 0, launch_mode: int = 0, mx_scaled_mfma: bool = False,
                 expert_activation: int = 0, group_pairs: int = 0):
        """expert_activation 1: hidden = relu(up)^2, ``gate`` must be None (a relu-squared bank has no gate descriptor).
        group_pairs: 1 = decode blocks serve up to four pairs of one expert, 0 = one pair per block (faster as measured)."""
        if (gate is None) != (expert_activation == 1):
            raise ValueError("the gate projection is absent exactly when expert_activation is 1")
        self._keep = (gate, up, down)
        self.top_k, self.max_tokens = top_k, max_tokens
        self.hidden = up.neuron_len
        self.intermediate = up.out_per_expert
        self.x_dtype, self.out_dtype = x_dtype, out_dtype
        config = L.MoeFfnConfig()
        if gate is not None:
            config.gate = gate.struct
        config.up, config.down = up.struct, down.struct
        config.expert_activation = expert_activation
        config.top_k, config.max_tokens = top_k, max_tokens
        config.x_dtype, config.out_dtype = _DTYPES[x_dtype], _DTYPES[out_dtype]
        config.swiglu_limit = swiglu_limit
        config.decode_token_limit = decode_token_limit
        config.launch_mode = launch_mode
        config.mx_scaled_mfma = int(mx_scaled_mfma)
        config.group_pairs = group_pairs
        handle = C.c_void_p()
        L.check(L.lib().mfq_amd_moe_ffn_create(C.byref(config), C.byref(handle)))
        self._handle = handle

    def run(self, x: torch.Tensor, ids: torch.Tensor, route_weights: torch.Tensor,
            out: torch.Tensor | None = None) -> torch.Tensor:
        if x.dtype != self.x_dtype:
            raise ValueError(f"x must be {self.x_dtype}")
        x, ids, route_weights = x.contiguous(), ids.contiguous(), route_weights.contiguous()
        tokens = x.shape[0]
        if out is None:
            out = torch.empty((tokens, self.hidden), dtype=self.out_dtype, device="cuda")
        L.check(L.lib().mfq_amd_moe_ffn_run(self._handle, x.data_ptr(), ids.data_ptr(), route_weights.data_ptr(),
                                            tokens, out.data_ptr(), _stream()))
        return out

    def run_logits(self, x: torch.Tensor, logits: torch.Tensor, out: torch.Tensor | None = None, normalize: bool = True,
                   norm_floor: float = 1e-20, scale: float = 1.0) -> torch.Tensor:
        """Top-k routing and the layer in one call (routing is fused into the plan kernel for decode batches)."""
        if x.dtype != self.x_dtype:
            raise ValueError(f"x must be {self.x_dtype}")
        x, logits = x.contiguous(), logits.contiguous()
        tokens = x.shape[0]
        if out is None:
            out = torch.empty((tokens, self.hidden), dtype=self.out_dtype, device="cuda")
        L.check(L.lib().mfq_amd_moe_ffn_run_logits(self._handle, x.data_ptr(), logits.data_ptr(), _dtype_code(logits),
                                                   int(normalize), norm_floor, scale, tokens, out.data_ptr(), _stream()))
        return out

    def run_router(self, x: torch.Tensor, router: torch.Tensor, out: torch.Tensor | None = None, normalize: bool = True,
                   norm_floor: float = 1e-20, scale: float = 1.0) -> torch.Tensor:
        """Router matmul, top-k routing and the layer in one call."""
        if x.dtype != self.x_dtype:
            raise ValueError(f"x must be {self.x_dtype}")
        x, router = x.contiguous(), router.contiguous()
        tokens = x.shape[0]
        if out is None:
            out = torch.empty((tokens, self.hidden), dtype=self.out_dtype, device="cuda")
        L.check(L.lib().mfq_amd_moe_ffn_run_router(self._handle, x.data_ptr(), router.data_ptr(), _dtype_code(router),
                                                   int(normalize), norm_floor, scale, tokens, out.data_ptr(), _stream()))
        return out

    def set_shared(self, gate: MixedMoeRuntime | None, up: MixedMoeRuntime, down: MixedMoeRuntime,
                   shared_activation: int = 0) -> None:
        """The layer's shared expert: dense one-expert projections (``MixedMoeRuntime.from_dense``); ``gate`` is None for
        the relu-squared activation."""
        self._shared_keep = (gate, up, down)
        first = lambda runtime: C.byref(runtime.struct.pools[0]) if runtime is not None else None
        L.check(L.lib().mfq_amd_moe_ffn_set_shared(self._handle, first(gate), first(up), first(down), shared_activation))

    def run_shared(self, x: torch.Tensor, ids: torch.Tensor, route_weights: torch.Tensor, shared_gate: torch.Tensor,
                   out: torch.Tensor | None = None) -> torch.Tensor:
        """run() plus the shared expert: out = half(routed) + shared_ffn(x) * shared_gate[token]; ``shared_gate`` holds one
        evaluated gate value per token (float32, float16 or bfloat16)."""
        if x.dtype != self.x_dtype:
            raise ValueError(f"x must be {self.x_dtype}")
        x, ids, route_weights, shared_gate = x.contiguous(), ids.contiguous(), route_weights.contiguous(), shared_gate.contiguous()
        tokens = x.shape[0]
        if shared_gate.numel() != tokens:
            raise ValueError("one shared gate value per token")
        if out is None:
            out = torch.empty((tokens, self.hidden), dtype=self.out_dtype, device="cuda")
        L.check(L.lib().mfq_amd_moe_ffn_run_shared(self._handle, x.data_ptr(), ids.data_ptr(), route_weights.data_ptr(),
                                                   shared_gate.data_ptr(), _dtype_code(shared_gate), tokens, out.data_ptr(), _stream()))
        return out

    def mx_scaled_slots(self) -> int:
        """Bit s set: the MXFP4 prefill tiles of projection s (gate, up, down) run on the block-scaled MFMA."""
        mask = C.c_int32(0)
        L.check(L.lib().mfq_amd_moe_ffn_mx_scaled_slots(self._handle, C.byref(mask)))
        return int(mask.value)

    def routes(self, tokens: int) -> tuple[torch.Tensor, torch.Tensor]:
        """Copies of the ids and weights the last run_logits selected."""
        ids, weights = C.c_void_p(), C.c_void_p()
        L.check(L.lib().mfq_amd_moe_ffn_routes(self._handle, C.byref(ids), C.byref(weights)))
        torch.cuda.synchronize()
        host_ids = np.empty(tokens * self.top_k, dtype=np.int32)
        host_weights = np.empty(tokens * self.top_k, dtype=np.float32)
        _memcpy_d2h(host_ids, ids.value)
        _memcpy_d2h(host_weights, weights.value)
        return (torch.from_numpy(host_ids.reshape(tokens, self.top_k)), torch.from_numpy(host_weights.reshape(tokens, self.top_k)))

    def run_raw(self, x_ptr: int, ids_ptr: int, weights_ptr: int, tokens: int, out_ptr: int, stream: int) -> None:
        L.check(L.lib().mfq_amd_moe_ffn_run(self._handle, x_ptr, ids_ptr, weights_ptr, tokens, out_ptr, stream))

    def stage_buffers(self, tokens: int) -> tuple[torch.Tensor, torch.Tensor]:
        """Copies of the last run's gate/up ``[T, k, 2, I]`` and pair ``[T, k, H]`` fp16 buffers."""
        gu, pairs = C.c_void_p(), C.c_void_p()
        L.check(L.lib().mfq_amd_moe_ffn_buffers(self._handle, C.byref(gu), C.byref(pairs)))
        torch.cuda.synchronize()
        n_gu = tokens * self.top_k * 2 * self.intermediate
        n_pairs = tokens * self.top_k * self.hidden
        host_gu = np.empty(n_gu, dtype=np.float16)
        host_pairs = np.empty(n_pairs, dtype=np.float16)
        _memcpy_d2h(host_gu, gu.value)
        _memcpy_d2h(host_pairs, pairs.value)
        return (host_gu.reshape(tokens, self.top_k, 2, self.intermediate),
                host_pairs.reshape(tokens, self.top_k, self.hidden))

    def enable_timing(self, enable: bool = True) -> None:
        L.check(L.lib().mfq_amd_moe_ffn_enable_timing(self._handle, int(enable)))

    def stage_times(self) -> dict:
        """Milliseconds of the last run's stages (needs enable_timing)."""
        ms = (C.c_float * 5)()
        L.check(L.lib().mfq_amd_moe_ffn_stage_times(self._handle, ms))
        return dict(zip(("plan", "gate_up", "swiglu", "down", "reduce"), (float(v) for v in ms)))

    def empty_bracket_ms(self) -> float:
        """Milliseconds between two events recorded back to back behind the last stage of the last run."""
        ms = C.c_float(0.0)
        L.check(L.lib().mfq_amd_moe_ffn_empty_bracket_ms(self._handle, C.byref(ms)))
        return float(ms.value)

    def touched_bytes(self) -> tuple[int, int]:
        nbytes, distinct = C.c_int64(), C.c_int32()
        L.check(L.lib().mfq_amd_moe_ffn_touched_bytes(self._handle, C.byref(nbytes), C.byref(distinct)))
        return nbytes.value, distinct.value

    def __del__(self):
        handle, self._handle = getattr(self, "_handle", None), None
        if handle and L is not None and getattr(L, "_lib", None) is not None:
            L._lib.mfq_amd_moe_ffn_destroy(handle)


def _memcpy_d2h(dst: np.ndarray, src_ptr: int) -> None:
    staging = torch.empty(dst.nbytes, dtype=torch.uint8, device="cuda")
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    status = hip.hipMemcpy(staging.data_ptr(), src_ptr, dst.nbytes, 3)   # device to device
    if status:
        raise RuntimeError(f"hipMemcpy failed: {status}")
    dst.view(np.uint8)[:] = staging.cpu().numpy()


def swiglu(gate: torch.Tensor, up: torch.Tensor, swiglu_limit: float = 0.0) -> torch.Tensor:
    gate, up = gate.contiguous(), up.contiguous()
    out = torch.empty_like(gate)
    L.check(L.lib().mfq_amd_swiglu(gate.data_ptr(), up.data_ptr(), gate.numel(), swiglu_limit, out.data_ptr(), _stream()))
    return out


def moe_weighted_reduce_shared_gate(pairs: torch.Tensor, weights: torch.Tensor, shared: torch.Tensor,
                                    gate_logits: torch.Tensor) -> torch.Tensor:
    """half(half(sum_r w * pair) + sigmoid(gate_logits[token]) * shared): pairs f16 [T, k, W], shared f16 [T, W]."""
    pairs, weights, shared, gate_logits = pairs.contiguous(), weights.contiguous(), shared.contiguous(), gate_logits.contiguous()
    tokens, k, width = pairs.shape
    out = torch.empty((tokens, width), dtype=torch.float16, device="cuda")
    L.check(L.lib().mfq_amd_weighted_reduce_shared_gate(pairs.data_ptr(), weights.data_ptr(), shared.data_ptr(),
                                                        gate_logits.data_ptr(), tokens, k, width, out.data_ptr(), _stream()))
    return out


def moe_add_shared_gate(routed: torch.Tensor, shared: torch.Tensor, gate_logits: torch.Tensor) -> torch.Tensor:
    """half(routed + sigmoid(gate_logits[row]) * shared), all f16 [rows, W]."""
    routed, shared, gate_logits = routed.contiguous(), shared.contiguous(), gate_logits.contiguous()
    rows, width = routed.shape
    out = torch.empty((rows, width), dtype=torch.float16, device="cuda")
    L.check(L.lib().mfq_amd_add_shared_gate(routed.data_ptr(), shared.data_ptr(), gate_logits.data_ptr(), rows, width,
                                            out.data_ptr(), _stream()))
    return out


def moe_weighted_reduce(pairs: torch.Tensor, weights: torch.Tensor, out_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    pairs, weights = pairs.contiguous(), weights.contiguous()
    tokens, k, width = pairs.shape
    out = torch.empty((tokens, width), dtype=out_dtype, device="cuda")
    L.check(L.lib().mfq_amd_weighted_reduce(pairs.data_ptr(), weights.data_ptr(), tokens, k, width, out.data_ptr(),
                                            _DTYPES[out_dtype], _stream()))
    return out
