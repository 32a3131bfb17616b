"""GPU parity of the paths the other files leave out: the tall instantiations of the streaming GEMV, the clamped
SwiGLU through decode and prefill, a dense one-expert FFN (the shared expert) feeding the shared-gate epilogue, a
NINT pool with per-row code widths inside a MoE layer, the uniform NINT4 layer at full size, and token counts at
and beyond the largest decode plan."""

import ctypes as C

import numpy as np
import pytest

from helpers import OracleMoeTensor, oracle_layer, rel_l2
from oracle import oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-3


# rows x ceil(batch / tokens per block) decides the instantiation (ops_dense.hip, GemvFastLaunch::run):
# at least 16384 (NVQ) / 32768 (others) takes the tall one: 8 row slots per wave for rows wider than 2048 columns,
# 16 for rows of 513..2048 columns, 8 four-row slots for rows of at most 512 columns.
@pytest.mark.parametrize("fmt,rows,width,batch", [
    ("NVQ3", 4096, 4096, 8), ("NVQ3", 4096, 4096, 16), ("NVQ3J-L", 4096, 4096, 9),      # two slabs, two tokens per block
    ("NINT4-32", 4096, 4096, 8), ("MXFP4", 4096, 4096, 8), ("NINT3", 4096, 2560, 9),    # two slabs, one token per block
    ("NINT4", 2048, 2048, 16), ("NVQ3J-L", 2048, 2048, 8), ("MXFP4", 2048, 1024, 16), ("NINT8", 2100, 1536, 16),
    ("NINT2", 2048, 512, 16), ("NINT4", 2050, 512, 16), ("NVQ3J-L", 2048, 512, 8), ("MXFP4", 4096, 256, 8),
    ("NINT4-32", 4096, 4096, 1), ("NVQ3", 4096, 4096, 1),        # the two dense benchmark matrices at batch 1 (not tall)
])
def test_tall_gemv_instantiations_vs_oracle(fmt, rows, width, batch):
    import torch
    from mfq_amd import _lib as L
    import benchdata
    import synth
    print("case", fmt, rows, width, batch, flush=True)
    tensor = benchdata.DeviceMoeTensor(f"test/tall/{fmt}/{rows}/{width}", 1, rows, width, [fmt])
    view = tensor.pools[0].view
    threshold = 16384 if fmt.startswith("NVQ") else 32768
    group = 2 if fmt.startswith("NVQ") and width > 2048 else 1
    assert batch == 1 or rows * ((batch + group - 1) // group) >= threshold, "the case must reach the tall instantiation"
    x = synth.to_bf16(synth.normal(f"test/tall/x/{width}/{batch}", (batch, width)))
    xd = torch.from_numpy(x).to(torch.bfloat16).cuda()
    y = torch.full((batch, rows), float("nan"), dtype=torch.float32, device="cuda")
    L.check(L.lib().mfq_amd_gemv(C.byref(view), 0, xd.data_ptr(), L.BF16, batch, width, y.data_ptr(), rows,
                                 torch.cuda.current_stream().cuda_stream))
    got = y.cpu().numpy()
    expect = O.Projection(tensor.host_layout(0)).rows(x, order=0)
    assert np.isfinite(got).all()
    err = rel_l2(got, expect)
    print(f"tall gemv {fmt} {rows}x{width} b{batch}: rel-L2 {err:.3e}")
    assert err <= TOL
    for b in range(batch):
        assert rel_l2(got[b], expect[b]) <= TOL


def test_clamped_swiglu_operator_vs_oracle():
    """swiglu_limit > 0 (mfq/kernels/cuda/mfe_ffn.h:111-114): the device's expf and the host's differ by an ulp of
    fp32 at most, so results agree to one fp16 step; values that do not touch the exponential agree exactly."""
    import torch
    from mfq_amd import runtime as R
    rng = np.random.default_rng(31)
    g = rng.normal(0, 4, 8192).astype(np.float16)
    u = rng.normal(0, 4, 8192).astype(np.float16)
    g[:6] = [20.0, -20.0, 7.0, 7.01, 0.0, -0.0]
    u[:6] = [9.0, -9.0, 7.0, -7.01, 3.0, 3.0]
    for limit in (7.0, 1.5, 30.0):
        got = R.swiglu(torch.from_numpy(g).cuda(), torch.from_numpy(u).cuda(), limit).cpu().numpy()
        expect = O.swiglu_array(g, u, limit)
        # fp16 bits on one ordered scale; zeros are compared by their bits, sign included (a gate of -0.0 gives -0.0 * up)
        ordered = lambda h: np.where(h.view(np.uint16) & 0x8000, -(h.view(np.uint16) & 0x7FFF).astype(np.int32),
                                     h.view(np.uint16).astype(np.int32))
        a, b = ordered(got), ordered(expect)
        assert np.all(np.abs(a - b) <= 1), (limit, np.abs(a - b).max())
        assert np.mean(got.view(np.uint16) == expect.view(np.uint16)) > 0.98
        zero = (expect.view(np.uint16) & 0x7FFF) == 0
        assert zero.sum() >= 2 and np.array_equal(got.view(np.uint16)[zero], expect.view(np.uint16)[zero])
        assert np.array_equal(got.view(np.uint16)[:6], expect.view(np.uint16)[:6])     # the six special inputs, bit for bit
        # the gate is clipped from above only, the other operand on both sides
        big = np.abs(got.astype(np.float32)).max()
        assert big <= limit * limit * 1.001


@pytest.mark.parametrize("tokens", [3, 16, 48])     # decode kernels (one wave and half a wave per token in the plan) and the tile kernels
def test_layer_with_clamped_swiglu_vs_oracle(tokens):
    import torch
    from mfq_amd import runtime as R
    import synth
    from test_gpu_moe import ALL_FORMATS, _inputs, _layer
    experts, hidden, inter, k = 24, 512, 128, 6
    tensors, runtimes, _ = _layer("test/moe/random", experts, hidden, inter, "random")
    x, ids, weights = _inputs(f"test/moe/clamp/in/{tokens}", tokens, experts, hidden, k)
    x = synth.to_bf16(x * 6.0)                      # gate/up values of a few units, so that the limit bites
    args = (torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda())
    limit = 1.0
    out = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=64, swiglu_limit=limit).run(*args).cpu().numpy()
    free = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=64).run(*args).cpu().numpy()
    expect = oracle_layer(x, ids, weights, tensors, swiglu_limit=limit)
    err = rel_l2(out, expect)
    print(f"clamped SwiGLU T={tokens}: rel-L2 {err:.3e}; distance to the unclamped layer {rel_l2(free, expect):.3e}")
    assert err <= TOL
    assert rel_l2(free, expect) > 0.05, "the limit must change the result, or the test shows nothing"


@pytest.mark.parametrize("tokens", [2, 16, 48])     # decode kernels (fused and separate activation) and the tile kernels
def test_layer_with_relu_squared_experts_vs_oracle(tokens):
    """expert_activation == 1 (mfq/kernels/cuda/mfe_ffn.h:79-82, :107-110): hidden = half(relu(up)^2), the bank has no
    gate projection."""
    import torch
    from mfq_amd import runtime as R
    from test_gpu_moe import _inputs, _layer
    experts, hidden, inter, k = 24, 512, 128, 6
    tensors, runtimes, _ = _layer("test/moe/random", experts, hidden, inter, "random")
    x, ids, weights = _inputs(f"test/moe/relu2/in/{tokens}", tokens, experts, hidden, k)
    args = (torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda())
    ffn = R.MfeFfnRuntime(None, runtimes[1], runtimes[2], top_k=k, max_tokens=64, expert_activation=1)
    out = ffn.run(*args).cpu().numpy()
    expect = oracle_layer(x, ids, weights, (None, tensors[1], tensors[2]), activation=1)
    gated = oracle_layer(x, ids, weights, tensors)
    err = rel_l2(out, expect)
    print(f"relu^2 experts T={tokens}: rel-L2 {err:.3e}; distance to the gated layer {rel_l2(gated, expect):.3e}")
    assert err <= TOL
    assert rel_l2(gated, expect) > 0.5
    with pytest.raises((ValueError, RuntimeError)):
        R.MfeFfnRuntime(runtimes[0], runtimes[1], runtimes[2], top_k=k, max_tokens=64, expert_activation=1)


@pytest.mark.parametrize("tokens,gate_dtype,activation", [(3, "f32", 0), (16, "f16", 0), (48, "bf16", 0), (5, "f32", 1)])
def test_layer_with_shared_expert_inside_the_ffn(tokens, gate_dtype, activation):
    """MfeFfnBatch::shared (mfq/kernels/cuda/mfe_ffn.h:45,60): routed experts and a dense shared expert in one call, the
    epilogue of mfq/kernels/cuda/mfe_ffn_device.cuh:1249-1263.  Expectation: the oracle's routed sum and the oracle's
    expert FFN of the shared projections, joined by two IEEE fp32 operations."""
    import torch
    from mfq_amd import runtime as R
    import synth
    from test_gpu_moe import _inputs, _layer
    experts, hidden, inter, shared_inter, k = 24, 512, 128, 192, 6
    tensors, runtimes, _ = _layer("test/moe/random", experts, hidden, inter, "random")
    rng = np.random.default_rng(77)
    dense = [synth.random_weights(fmt, rows, width, rng) for fmt, rows, width in
             (("NINT4", shared_inter, hidden), ("NVQ3J-L", shared_inter, hidden), ("MXFP4", hidden, shared_inter))]
    shared = [R.MixedMoeRuntime.from_dense(t) for t in dense]
    x, ids, weights = _inputs(f"test/moe/shared/in/{tokens}", tokens, experts, hidden, k)
    gate32 = rng.uniform(0.05, 0.95, tokens).astype(np.float32)
    if gate_dtype == "f16":
        gate_host, gate_dev = gate32.astype(np.float16), torch.from_numpy(gate32.astype(np.float16)).cuda()
    elif gate_dtype == "bf16":
        gate_host = synth.to_bf16(gate32)
        gate_dev = torch.from_numpy(gate_host).to(torch.bfloat16).cuda()
    else:
        gate_host, gate_dev = gate32, torch.from_numpy(gate32).cuda()
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=64)
    ffn.set_shared(None if activation else shared[0], shared[1], shared[2], activation)
    out = ffn.run_shared(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda(),
                         gate_dev).cpu().numpy()
    routed = oracle_layer(x, ids, weights, tensors)
    g, u, d = (O.Projection(O.runtime_layout(t)) for t in dense)
    shared_out = O.expert_ffn(g, u, d, x, 0, 0.0, activation).astype(np.float16)
    expect = O.shared_expert_epilogue(routed, shared_out, gate_host)
    err = rel_l2(out, expect)
    print(f"shared expert inside the FFN T={tokens} gate {gate_dtype} activation {activation}: rel-L2 {err:.3e}; "
          f"share of the shared expert {rel_l2(routed, expect):.3e}")
    assert err <= TOL
    assert rel_l2(routed, expect) > 0.05


@pytest.mark.parametrize("tokens", [5, 16, 40])      # small and sorted decode plans, prefill tiles
def test_layer_with_absent_and_repeated_routes(tokens):
    """Routes whose expert id lies outside [0, experts) add nothing (cuda/ops/moe.cpp:257-320 skips them in the plan),
    and a token may name one expert twice (two pairs of one expert and token).  Also: an empty batch is a no-op, and a
    batch of exactly max_tokens runs."""
    import torch
    from mfq_amd import runtime as R
    from test_gpu_moe import _inputs, _layer
    experts, hidden, inter, k = 24, 512, 128, 6
    tensors, runtimes, _ = _layer("test/moe/random", experts, hidden, inter, "random")
    x, ids, weights = _inputs(f"test/moe/edge/in/{tokens}", tokens, experts, hidden, k)
    ids = ids.copy()
    rng = np.random.default_rng(tokens)
    absent = rng.random(ids.shape) < 0.2
    ids[absent] = np.where(rng.random(int(absent.sum())) < 0.5, -1, experts + 3)
    repeated = (rng.random(tokens) < 0.5) & ~absent[:, 0] & ~absent[:, 1]
    ids[repeated, 1] = ids[repeated, 0]
    assert absent.any() and repeated.any()
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=tokens)          # the batch fills the workspace exactly
    xd = torch.from_numpy(x).to(torch.bfloat16).cuda()
    out = ffn.run(xd, torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda()).cpu().numpy()
    # the oracle sees the absent routes as routes of expert 0 with weight zero
    seen_ids, seen_weights = np.where(absent, 0, ids).astype(np.int32), np.where(absent, 0.0, weights).astype(np.float32)
    expect = oracle_layer(x, seen_ids, seen_weights, tensors)
    err = rel_l2(out, expect)
    print(f"absent and repeated routes T={tokens}: rel-L2 {err:.3e} ({int(absent.sum())} absent, {int(repeated.sum())} repeated)")
    assert err <= TOL
    # a token whose routes are all absent gets zeros
    none = np.full_like(ids, -1)
    zeros = ffn.run(xd, torch.from_numpy(none).cuda(), torch.from_numpy(weights).cuda()).cpu().numpy()
    assert not zeros.any()
    # an empty batch leaves the output untouched and reports success
    marker = torch.full((1, hidden), 7.0, dtype=torch.float32, device="cuda")
    ffn.run(xd[:0], torch.from_numpy(ids[:0]).cuda(), torch.from_numpy(weights[:0]).cuda(), marker[:0])
    assert float(marker.min()) == 7.0
    with pytest.raises((ValueError, RuntimeError)):
        R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=tokens - 1).run(xd, torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda())


@pytest.mark.parametrize("fmt", ["NINT4", "NVQ3J-L", "MXFP4", "NINT3-odd"])
@pytest.mark.parametrize("tokens", [4, 40])
def test_dense_single_expert_ffn_feeds_the_shared_gate_epilogue(fmt, tokens):
    """The shared expert: one dense pool per projection (no expert map), every token routed to it with weight 1,
    fp16 output; then out = half(routed + sigmoid(gate) * shared) (mfq/kernels/cuda/moe.cu:1557-1571)."""
    import torch
    from mfq_amd import runtime as R
    import synth
    hidden, inter = (512, 128) if fmt != "NINT3-odd" else (200, 72)      # the odd widths take the exact decoders
    name = "NINT3" if fmt == "NINT3-odd" else fmt
    rng = np.random.default_rng(5)
    dense = [synth.random_weights(name, rows, width, rng) for rows, width in ((inter, hidden), (inter, hidden), (hidden, inter))]
    runtimes = [R.MixedMoeRuntime.from_dense(t) for t in dense]
    assert all(r.experts == 1 and r.pools[0].view.expert_local is None for r in runtimes)
    x = synth.to_bf16(synth.normal(f"test/shared/x/{tokens}/{hidden}", (tokens, hidden)))
    ids = np.zeros((tokens, 1), dtype=np.int32)
    ones = np.ones((tokens, 1), dtype=np.float32)
    ffn = R.MfeFfnRuntime(*runtimes, top_k=1, max_tokens=64, out_dtype=torch.float16)
    shared = ffn.run(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(ones).cuda())
    projections = tuple(O.Projection(O.runtime_layout(t)) for t in dense)
    shared_expect = O.moe_layer(x, ids, ones, lambda e: projections)
    err = rel_l2(shared.cpu().numpy().astype(np.float32), shared_expect)
    print(f"shared expert {fmt} T={tokens}: rel-L2 {err:.3e}")
    assert err <= TOL
    routed = rng.normal(0, 0.05, (tokens, hidden)).astype(np.float16)
    gate = rng.normal(0, 2, tokens).astype(np.float32)
    out = R.moe_add_shared_gate(torch.from_numpy(routed).cuda(), shared, torch.from_numpy(gate).cuda()).cpu().numpy()
    expect = O.weighted_reduce_shared_gate(routed[:, None, :], ones, shared_expect.astype(np.float16), gate)
    assert rel_l2(out.astype(np.float32), expect.astype(np.float32)) <= TOL
    # and bit for bit on the device's own shared rows
    same = O.weighted_reduce_shared_gate(routed[:, None, :], ones, shared.cpu().numpy(), gate)
    assert np.array_equal(out.view(np.uint16), same.view(np.uint16))


@pytest.mark.parametrize("tokens", [5, 60])
def test_layer_with_a_pool_of_per_row_code_widths(tokens):
    """A NINT pool whose rows have different code widths (uniform_bits = 0: the exact decoders read the per-row
    widths and bit offsets) beside streaming pools in one layer."""
    import torch
    from mfq_amd import runtime as R
    import synth
    from mfq_amd.formats import mfe as MFE, nint as FN, nvq as FV
    from mfq_amd.quantize import nint_quant as QN, nvq_quant as QV
    experts, hidden, inter, k = 9, 256, 96, 3
    rng = np.random.default_rng(41)

    def tensor(out, width):
        mixed = rng.integers(1, 9, 3 * out).astype(np.uint8)
        pools = [
            MFE.MfePool(np.array([0, 4, 8], dtype=np.int32), synth.random_weights("NINT4", 3 * out, width, rng)),
            MFE.MfePool(np.array([1, 2, 6], dtype=np.int32), QN.random_codes(3 * out, width, FN.NintSpec(4, 24, 6), rng, row_q_bits=mixed)),
            MFE.MfePool(np.array([3, 5, 7], dtype=np.int32), synth.random_weights("NVQ3J-L", 3 * out, width, rng)),
        ]
        return MFE.MfeTensor((experts, out, width), pools)

    tensors = [tensor(inter, hidden), tensor(inter, hidden), tensor(hidden, inter)]
    # bring the mixed-width pool's weights to the scale of the others, so that no fp16 stage overflows
    for t in tensors:
        pool = t.pools[1].tensor
        pool.neuron_scale = np.full_like(pool.neuron_scale, np.float32(np.float16(0.00002)), dtype=np.float32)
        pool.neuron_min = np.full_like(pool.neuron_min, np.float32(np.float16(0.0005)), dtype=np.float32)
    runtimes = [R.MixedMoeRuntime(t) for t in tensors]
    assert runtimes[0].pools[1].view.uniform_bits == 0
    x = synth.to_bf16(synth.normal(f"test/mixedq/x/{tokens}", (tokens, hidden)))
    ids = np.stack([np.random.default_rng(100 + t).permutation(experts)[:k] for t in range(tokens)]).astype(np.int32)
    weights = np.random.default_rng(7).uniform(0.1, 0.5, (tokens, k)).astype(np.float32)
    out = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=64).run(
        torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda()).cpu().numpy()
    expect = oracle_layer(x, ids, weights, tensors)
    assert np.isfinite(expect).all() and np.abs(expect).max() > 0
    err = rel_l2(out, expect)
    print(f"per-row widths T={tokens}: rel-L2 {err:.3e}")
    assert err <= TOL


@pytest.mark.parametrize("tokens", [1, 4, 16])
def test_uniform_nint4_layer_at_full_size_vs_oracle(tokens):
    """512 experts x (2048 <-> 512), every projection NINT4 with 24-column groups, top-10, softmax routing."""
    import torch
    from mfq_amd import runtime as R
    import benchdata
    import synth
    experts, hidden, inter, k = 512, 2048, 512, 10
    if "layer" not in _UNIFORM:
        _UNIFORM["layer"] = benchdata.device_layer("test/cfg3/layer", experts, hidden, inter, [["NINT4"] * experts] * 3)
    layer = _UNIFORM["layer"]
    x = synth.to_bf16(synth.normal(f"test/cfg3/x/{tokens}", (tokens, hidden)))
    router = synth.to_bf16(synth.normal("test/cfg3/router", (experts, hidden), 0.02))
    xd = torch.from_numpy(x).to(torch.bfloat16).cuda()
    logits = R.router_logits(xd, torch.from_numpy(router).to(torch.bfloat16).cuda())
    ffn = R.MfeFfnRuntime(*layer, top_k=k, max_tokens=16)
    out = ffn.run_logits(xd, logits).cpu().numpy()
    ids, weights = (t.numpy() for t in ffn.routes(tokens))
    ids_ref, weights_ref = O.topk(O.router_logits(x, router), k)
    assert np.array_equal(ids, ids_ref)
    cache = {}

    def of(expert):
        if expert not in cache:
            cache[expert] = tuple(O.Projection(t.host_layout(expert)) for t in layer)
        return cache[expert]
    expect = O.moe_layer(x, ids_ref, weights_ref, of)
    err = rel_l2(out, expect)
    print(f"cfg3 uniform NINT4 T={tokens}: rel-L2 {err:.3e}")
    assert err <= TOL


_UNIFORM = {}


@pytest.mark.parametrize("tokens", [102, 103, 128])
def test_token_counts_around_the_largest_decode_plan(tokens):
    """decode_token_limit = 128 with top-10 is clamped to 102 tokens (1020 pairs, one plan thread per pair): 102
    tokens run the decode kernels, more run the grouped GEMM."""
    import torch
    from mfq_amd import _lib as L, runtime as R
    import synth
    from test_gpu_moe import _layer
    experts, hidden, inter, k = 24, 256, 64, 10
    assert L.lib().mfq_amd_moe_ffn_decode_limit(128, k) == 102
    tensors, runtimes, _ = _layer("test/moe/limit", experts, hidden, inter, "random")
    x = synth.to_bf16(synth.normal(f"test/limit/x/{tokens}", (tokens, hidden)))
    ids = np.stack([np.random.default_rng(300 + t).permutation(experts)[:k] for t in range(tokens)]).astype(np.int32)
    weights = np.full((tokens, k), 0.1, dtype=np.float32)
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=128, decode_token_limit=128)
    out = ffn.run(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda()).cpu().numpy()
    err = rel_l2(out, oracle_layer(x, ids, weights, tensors))
    print(f"T={tokens} with decode limit 128, top-10: rel-L2 {err:.3e}")
    assert err <= TOL


@pytest.mark.parametrize("case", ["uniform", "mixed", "f16", "ragged"])
def test_prefill_mxfp4_on_the_block_scaled_mfma(case):
    """mx_scaled_mfma = 1: prefill tiles of MXFP4 pools run on v_mfma_scale_f32_32x32x64_f8f6f4 with the weights as
    stored (fp4 + E8M0 block scales) and the activations as E4M3 terms that add up to the source exactly (two for
    bf16, three for fp16), the other formats on the fp16 tiles as before.  Same bar as every path: rel-L2 <= 1e-3."""
    import torch
    from mfq_amd import runtime as R
    import synth
    from test_gpu_moe import ALL_FORMATS, _layer
    experts, hidden, inter, k, tokens, dtype = 6, 512, 128, 3, 150, torch.bfloat16
    uniform, mix = None, ALL_FORMATS
    if case == "uniform":
        uniform = "MXFP4"
    elif case == "mixed":
        experts, k, tokens, mix = 24, 6, 300, (("MXFP4", 0.5), ("NINT4", 0.25), ("NVQ3J-L", 0.25))
    elif case == "f16":
        uniform, dtype = "MXFP4", torch.float16
    else:
        uniform, hidden, inter, tokens = "MXFP4", 96, 160, 70         # three and five lane blocks per row: odd counts
    tensors, runtimes, formats = _layer(f"test/mxscaled/{case}", experts, hidden, inter, "random", mix=mix, uniform=uniform)
    assert any("MXFP4" in f for f in formats)
    x = synth.normal(f"test/mxscaled/x/{case}", (tokens, hidden))
    x = x.astype(np.float16).astype(np.float32) if dtype == torch.float16 else synth.to_bf16(x)
    ids = synth.zipf_routes(f"test/mxscaled/ids/{case}", tokens, experts, k)
    weights = np.full((tokens, k), 1.0 / k, dtype=np.float32)
    args = (torch.from_numpy(x).to(dtype).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda())
    expect = oracle_layer(x, ids, weights, tensors)
    on = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=tokens, x_dtype=dtype, mx_scaled_mfma=True)
    off = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=tokens, x_dtype=dtype)
    # the switch took: every projection with MXFP4 experts is on the block-scaled kernel, none without the switch
    assert on.mx_scaled_slots() == sum(1 << s for s in range(3) if "MXFP4" in formats[s]) and off.mx_scaled_slots() == 0
    scaled = on.run(*args).cpu().numpy()
    plain = off.run(*args).cpu().numpy()
    err_scaled, err_plain = rel_l2(scaled, expect), rel_l2(plain, expect)
    print(f"MXFP4 prefill {case}: block-scaled MFMA {err_scaled:.3e}, fp16 tiles {err_plain:.3e}")
    assert np.isfinite(scaled).all()
    assert err_scaled <= TOL and err_plain <= TOL
