"""GPU parity of the mixed-format MoE FFN through the C ABI against the oracle's CPU expert
FFN (fp32 accumulate, fp16 stage rounding).  Tolerance: rel-L2 <= 1e-3 on the layer output."""

import numpy as np
import pytest

from helpers import OracleMoeTensor, oracle_layer, rel_l2
from oracle import oracle as O

pytestmark = pytest.mark.gpu

FFN_TOL = 1e-3
ALL_FORMATS = (("NINT2", 1 / 6), ("NINT3", 1 / 6), ("NINT4", 1 / 6), ("NINT8", 1 / 6), ("NVQ3J-L", 1 / 6), ("MXFP4", 1 / 6))


_LAYERS = {}


def _layer(tag, experts, hidden, inter, mode, mix=ALL_FORMATS, uniform=None):
    from mfq_amd import runtime as R
    import synth
    key = (tag, experts, hidden, inter, mode, uniform)
    if key not in _LAYERS:
        tensors, formats = synth.build_layer(tag, experts, hidden, inter, mix=mix, mode=mode, uniform=uniform)
        _LAYERS[key] = (tensors, [R.MixedMoeRuntime(t) for t in tensors], formats)
    return _LAYERS[key]


def _inputs(tag, tokens, experts, hidden, k):
    import synth
    x = synth.to_bf16(synth.normal(f"{tag}/x", (tokens, hidden)))
    router = synth.to_bf16(synth.normal(f"{tag}/router", (experts, hidden), 0.02))
    logits = O.router_logits(x, router)
    ids, weights = O.topk(logits, k)
    return x, ids, weights


@pytest.mark.parametrize("mode", ["random", "pack"])
@pytest.mark.parametrize("tokens", [1, 4, 16])
def test_decode_ffn_vs_oracle(mode, tokens):
    import torch
    from mfq_amd import runtime as R
    experts, hidden, inter, k = (24, 512, 128, 6) if mode == "random" else (12, 256, 64, 4)
    tensors, runtimes, formats = _layer(f"test/moe/{mode}", experts, hidden, inter, mode)
    x, ids, weights = _inputs(f"test/moe/in/{tokens}", tokens, experts, hidden, k)
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=16)
    out = ffn.run(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(),
                  torch.from_numpy(weights).cuda()).cpu().numpy()
    expect = oracle_layer(x, ids, weights, tensors)
    err = rel_l2(out, expect)
    print(f"decode {mode} T={tokens} rel-L2 {err:.3e}; formats used {sorted(set(sum(formats, [])))}")
    assert err <= FFN_TOL
    nbytes, distinct = ffn.touched_bytes()
    assert distinct == len(set(ids.reshape(-1).tolist()))
    assert nbytes > 0


@pytest.mark.parametrize("tokens", [2, 5, 12, 16])
def test_decode_blocks_that_serve_a_group_of_pairs_vs_oracle(tokens):
    """Few experts, many pairs, group_pairs = 1: the plan groups up to four neighbouring pairs of one expert and one block
    of the rows kernels multiplies for all of them (12 tokens x top-4 over 8 experts is six pairs per expert, i.e. groups
    of four and two).  Against the oracle, and bit for bit against the same layer with one block per pair: a pair's
    arithmetic does not depend on who shares its block."""
    import torch
    from mfq_amd import runtime as R
    experts, hidden, inter, k = 8, 512, 128, 4
    tensors, runtimes, _ = _layer("test/moe/groups", experts, hidden, inter, "random")
    x, ids, weights = _inputs(f"test/moe/groups/in/{tokens}", tokens, experts, hidden, k)
    if tokens >= 5:
        ids = ids.copy(); ids[1, 2] = -1                           # an unrouted pair among the groups
    args = (torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda())
    routed = ids >= 0
    results = {}
    for mode in (1, 0):
        ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=16, group_pairs=mode)
        out = ffn.run(*args).cpu().numpy()
        gu, pairs = ffn.stage_buffers(tokens)
        results[mode] = (out, np.asarray(gu).reshape(tokens, k, -1)[routed], np.asarray(pairs).reshape(tokens, k, -1)[routed])
    expect = oracle_layer(x, np.where(routed, ids, 0), np.where(routed, weights, 0.0).astype(np.float32), tensors)
    for mode, (out, gu, pairs) in results.items():
        err = rel_l2(out, expect)
        print(f"grouped decode T={tokens} mode {mode}: rel-L2 {err:.3e}")
        assert err <= FFN_TOL, mode
        assert np.array_equal(gu.view(np.uint16), results[0][1].view(np.uint16)), mode
        assert np.array_equal(pairs.view(np.uint16), results[0][2].view(np.uint16)), mode
        assert np.array_equal(out.view(np.uint32), results[0][0].view(np.uint32)), mode


def test_decode_stage_buffers_vs_oracle():
    """gate/up and per-pair down outputs, stage by stage."""
    import torch
    from mfq_amd import runtime as R
    experts, hidden, inter, k, tokens = 12, 256, 64, 4, 5
    tensors, runtimes, _ = _layer("test/moe/stages", experts, hidden, inter, "random")
    x, ids, weights = _inputs("test/moe/stages/in", tokens, experts, hidden, k)
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=8)
    ffn.run(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda())
    gu, pairs = ffn.stage_buffers(tokens)
    gate, up, down = (OracleMoeTensor(t) for t in tensors)
    for t in range(tokens):
        for r in range(k):
            e = int(ids[t, r])
            g = gate.projection(e).rows(x[t:t + 1])[0]
            u = up.projection(e).rows(x[t:t + 1])[0]
            assert rel_l2(gu[t, r, 0].astype(np.float32), g) < 2e-3   # one fp16 rounding
            assert rel_l2(gu[t, r, 1].astype(np.float32), u) < 2e-3
            full = O.expert_ffn(gate.projection(e), up.projection(e), down.projection(e), x[t:t + 1])[0]
            assert rel_l2(pairs[t, r].astype(np.float32), full) < 2e-3


@pytest.mark.parametrize("uniform", ["NINT4", "NVQ3J-L", "MXFP4", "NINT3"])
def test_uniform_layer(uniform):
    import torch
    from mfq_amd import runtime as R
    experts, hidden, inter, k, tokens = 16, 512, 128, 4, 4
    tensors, runtimes, _ = _layer(f"test/moe/uniform/{uniform}", experts, hidden, inter, "random", uniform=uniform)
    x, ids, weights = _inputs("test/moe/uniform/in", tokens, experts, hidden, k)
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=8)
    out = ffn.run(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(),
                  torch.from_numpy(weights).cuda()).cpu().numpy()
    assert rel_l2(out, oracle_layer(x, ids, weights, tensors)) <= FFN_TOL


@pytest.mark.parametrize("hidden,inter", [(2048, 512), (640, 96), (1024, 32), (96, 64), (160, 128)])
def test_decode_wide_rows(hidden, inter):
    """Rows wider than 512 columns use 64 lanes per row; 640 leaves lanes without a column block.  The narrow shapes
    have rows of two to eight groups: some classes then take their group levels as shared level words (at least
    four levels per row) and some by one load per lane, in the same launch."""
    import torch
    from mfq_amd import runtime as R
    experts, k, tokens = 12, 4, 3
    tensors, runtimes, _ = _layer(f"test/moe/wide/{hidden}", experts, hidden, inter, "random")
    x, ids, weights = _inputs(f"test/moe/wide/in/{hidden}", tokens, experts, hidden, k)
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=8)
    out = ffn.run(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(),
                  torch.from_numpy(weights).cuda()).cpu().numpy()
    err = rel_l2(out, oracle_layer(x, ids, weights, tensors))
    print(f"decode H={hidden} I={inter} rel-L2 {err:.3e}")
    assert err <= FFN_TOL


def test_streaming_and_exact_kernels_agree():
    """launch_mode 1 runs every pool on the exact decoders; both must match the oracle and each other."""
    import torch
    from mfq_amd import runtime as R
    experts, hidden, inter, k, tokens = 24, 512, 128, 6, 7
    tensors, runtimes, _ = _layer("test/moe/random", experts, hidden, inter, "random")
    x, ids, weights = _inputs("test/moe/modes", tokens, experts, hidden, k)
    args = (torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda())
    fast = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=8, launch_mode=0).run(*args).cpu().numpy()
    exact = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=8, launch_mode=1).run(*args).cpu().numpy()
    expect = oracle_layer(x, ids, weights, tensors)
    assert rel_l2(fast, expect) <= FFN_TOL and rel_l2(exact, expect) <= FFN_TOL
    assert rel_l2(fast, exact) <= FFN_TOL


def test_exact_kernels_serve_what_streaming_cannot():
    """f32 activations, and a width that is not a multiple of 32, take the exact decoders."""
    import torch
    from mfq_amd import runtime as R
    experts, k, tokens = 8, 3, 4
    mix = (("NINT2", 0.25), ("NINT3", 0.25), ("NINT4", 0.25), ("NINT8", 0.25))
    tensors, runtimes, _ = _layer("test/moe/odd", experts, 200, 72, "random", mix=mix)
    x, ids, weights = _inputs("test/moe/odd/in", tokens, experts, 200, k)
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=8)
    out = ffn.run(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(),
                  torch.from_numpy(weights).cuda()).cpu().numpy()
    assert rel_l2(out, oracle_layer(x, ids, weights, tensors)) <= FFN_TOL
    tensors, runtimes, _ = _layer("test/moe/random", 24, 512, 128, "random")
    x, ids, weights = _inputs("test/moe/f32", tokens, 24, 512, 6)
    ffn = R.MfeFfnRuntime(*runtimes, top_k=6, max_tokens=8, x_dtype=torch.float32)
    out = ffn.run(torch.from_numpy(x).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda()).cpu().numpy()
    assert rel_l2(out, oracle_layer(x, ids, weights, tensors)) <= FFN_TOL


@pytest.mark.parametrize("tokens", [4, 40])                 # the rows kernels and the tile kernels
def test_layer_with_the_4096_entry_e8_profile(tokens):
    """NVQ2J-XL experts (12-bit indices, codebooks read from global memory) beside streaming formats."""
    import torch
    from mfq_amd import runtime as R
    experts, hidden, inter, k = 12, 256, 96, 4
    mix = (("NVQ2J-XL", 0.5), ("NINT4", 0.25), ("NVQ3J-L", 0.25))
    tensors, runtimes, formats = _layer("test/moe/xl", experts, hidden, inter, "random", mix=mix)
    assert any("NVQ2J-XL" in f for f in formats)
    x, ids, weights = _inputs(f"test/moe/xl/in/{tokens}", tokens, experts, hidden, k)
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=tokens)
    out = ffn.run(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(),
                  torch.from_numpy(weights).cuda()).cpu().numpy()
    assert rel_l2(out, oracle_layer(x, ids, weights, tensors)) <= FFN_TOL


def test_tall_down_blocks_beside_pools_of_the_exact_kernels():
    """32 tokens x top-4 over 2048 outputs: 128 pairs x 8 down blocks of 256 rows reach the floor of the launch, and
    a pool that only the exact kernels serve keeps the SwiGLU in a kernel of its own, so the streaming pools run
    the sixteen-slot rows kernel on packed hidden rows."""
    import torch
    from mfq_amd import runtime as R
    experts, hidden, inter, k, tokens = 12, 2048, 96, 4, 32
    mix = (("NVQ2J-XL", 0.3), ("NINT4", 0.25), ("NVQ3J-L", 0.2), ("NINT3", 0.15), ("MXFP4", 0.1))
    tensors, runtimes, formats = _layer("test/moe/tall-down", experts, hidden, inter, "random", mix=mix)
    assert any("NVQ2J-XL" in f for f in formats) and len(set(sum(formats, []))) >= 3
    x, ids, weights = _inputs("test/moe/tall-down/in", tokens, experts, hidden, k)
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=tokens)
    out = ffn.run(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(),
                  torch.from_numpy(weights).cuda()).cpu().numpy()
    assert rel_l2(out, oracle_layer(x, ids, weights, tensors)) <= FFN_TOL


def test_many_pairs_per_expert_and_large_activations():
    """32 tokens over 6 experts: every expert serves many pairs; per-token activation scales from
    2^-3 to 2^5 exercise the per-token normalisation of the streaming kernels (larger inputs overflow
    the fp16 stage outputs of the reference chain itself, smaller ones push the hidden values into
    fp16 subnormals where one rounding flips whole percents)."""
    import torch
    from mfq_amd import runtime as R
    import synth
    experts, hidden, inter, k, tokens = 6, 256, 64, 3, 32
    tensors, runtimes, _ = _layer("test/moe/few", experts, hidden, inter, "random")
    x, ids, weights = _inputs("test/moe/few/in", tokens, experts, hidden, k)
    x = synth.to_bf16(x * np.exp2(np.linspace(-3.0, 5.0, tokens)).astype(np.float32)[:, None])
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=32)
    out = ffn.run(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(),
                  torch.from_numpy(weights).cuda()).cpu().numpy()
    expect = oracle_layer(x, ids, weights, tensors)
    for t in range(tokens):
        assert np.isfinite(expect[t]).all() and rel_l2(out[t], expect[t]) <= FFN_TOL, t


@pytest.mark.parametrize("tokens,experts,k", [(1, 24, 6), (16, 24, 6), (32, 128, 8), (5, 256, 8), (3, 8, 2), (40, 24, 6),
                                                (13, 40, 4), (9, 512, 10)])
def test_layer_with_fused_routing_equals_topk_then_layer(tokens, experts, k):
    """run_logits selects the routes inside the plan kernel (up to 32 tokens; 40 takes the top-k kernel):
    ids bit-equal to the stand-alone top-k, weights and output equal to the two-call sequence."""
    import torch
    from mfq_amd import runtime as R
    hidden, inter = 512, 128
    tensors, runtimes, _ = _layer(f"test/moe/fused/{experts}", experts, hidden, inter, "random")
    x, _, _ = _inputs(f"test/moe/fused/in/{tokens}", tokens, experts, hidden, k)
    rng = np.random.default_rng(tokens * 1000 + experts)
    logits = torch.from_numpy(rng.standard_normal((tokens, experts)).astype(np.float32)).to(torch.bfloat16).cuda()
    xd = torch.from_numpy(x).to(torch.bfloat16).cuda()
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=64)
    ids, weights = R.moe_topk(logits, k)
    want = ffn.run(xd, ids, weights).cpu().numpy()
    for _ in range(2):                                 # the second call reuses the object's route buffers
        got = ffn.run_logits(xd, logits).cpu().numpy()
        got_ids, got_weights = ffn.routes(tokens)
        np.testing.assert_array_equal(got_ids.numpy(), ids.cpu().numpy())
        np.testing.assert_array_equal(got_weights.numpy(), weights.cpu().numpy())
        np.testing.assert_array_equal(got, want)
    expect = oracle_layer(x, ids.cpu().numpy(), weights.cpu().numpy(), tensors)
    assert rel_l2(got, expect) <= FFN_TOL


@pytest.mark.parametrize("tokens", [1, 9, 48])
def test_layer_with_the_router_matmul_in_front(tokens):
    """run_router = router matmul + top-k + layer in one call: same routes and output as the three calls."""
    import torch
    from mfq_amd import runtime as R
    import synth
    experts, hidden, inter, k = 24, 512, 128, 6
    tensors, runtimes, _ = _layer("test/moe/random", experts, hidden, inter, "random")
    x = synth.to_bf16(synth.normal(f"test/moe/router/x/{tokens}", (tokens, hidden)))
    router = synth.to_bf16(synth.normal("test/moe/router/w", (experts, hidden), 0.02))
    xd = torch.from_numpy(x).to(torch.bfloat16).cuda()
    rd = torch.from_numpy(router).to(torch.bfloat16).cuda()
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=64)
    ids, weights = R.moe_topk(R.router_logits(xd, rd), k)
    want = ffn.run(xd, ids, weights).cpu().numpy()
    got = ffn.run_router(xd, rd).cpu().numpy()
    got_ids, got_weights = ffn.routes(tokens)
    ids_ref, weights_ref = O.topk(O.router_logits(x, router), k)
    np.testing.assert_array_equal(got_ids.numpy(), ids_ref)
    np.testing.assert_array_equal(got_ids.numpy(), ids.cpu().numpy())
    np.testing.assert_array_equal(got, want)
    assert rel_l2(got, oracle_layer(x, ids_ref, weights_ref, tensors)) <= FFN_TOL


def test_decode_layer_replayed_from_a_hip_graph():
    """The layer allocates nothing and synchronises nothing: captured once, every replay (with eager work and
    synchronisation in between) gives the eager result, for the id-based and the logits-based entry."""
    import torch
    from mfq_amd import runtime as R
    experts, hidden, inter, k, tokens = 24, 512, 128, 6, 8
    tensors, runtimes, _ = _layer("test/moe/random", experts, hidden, inter, "random")
    x, ids, weights = _inputs("test/moe/graph", tokens, experts, hidden, k)
    rng = np.random.default_rng(11)
    xd = torch.from_numpy(x).to(torch.bfloat16).cuda()
    idd, wd = torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda()
    logits = torch.from_numpy(rng.standard_normal((tokens, experts)).astype(np.float32)).to(torch.bfloat16).cuda()
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=16)
    eager_ids = ffn.run(xd, idd, wd).clone()
    eager_logits = ffn.run_logits(xd, logits).clone()
    out_ids = torch.empty_like(eager_ids)
    out_logits = torch.empty_like(eager_logits)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        ffn.run(xd, idd, wd, out_ids)                      # warm-up on the capture stream
        ffn.run_logits(xd, logits, out_logits)
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            ffn.run(xd, idd, wd, out_ids)
            ffn.run_logits(xd, logits, out_logits)
    for replay in range(3):
        out_ids.zero_(); out_logits.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_ids, eager_ids), f"replay {replay}: id-based entry differs from the eager run"
        assert torch.equal(out_logits, eager_logits), f"replay {replay}: logits-based entry differs from the eager run"
        _ = ffn.run(xd, idd, wd)                           # eager work between replays
    expect = oracle_layer(x, ids, weights, tensors)
    assert rel_l2(out_ids.cpu().numpy(), expect) <= FFN_TOL


@pytest.mark.parametrize("tokens", [40, 200])
def test_prefill_ffn_vs_oracle(tokens):
    """More tokens than the decode limit: route tiles through the MFMA grouped GEMM."""
    import torch
    from mfq_amd import runtime as R
    import synth
    experts, hidden, inter, k = 24, 512, 128, 6
    tensors, runtimes, _ = _layer("test/moe/random", experts, hidden, inter, "random")
    x = synth.to_bf16(synth.normal(f"test/prefill/x/{tokens}", (tokens, hidden)))
    ids = synth.zipf_routes(f"test/prefill/ids/{tokens}", tokens, experts, k)
    weights = np.full((tokens, k), 1.0 / k, dtype=np.float32)
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=256)
    out = ffn.run(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(),
                  torch.from_numpy(weights).cuda()).cpu().numpy()
    expect = oracle_layer(x, ids, weights, tensors)
    err = rel_l2(out, expect)
    print(f"prefill T={tokens} rel-L2 {err:.3e}")
    assert err <= FFN_TOL


@pytest.mark.parametrize("mode,hidden,inter,tokens,experts,k", [
    ("pack", 512, 128, 300, 24, 6),       # uniform code widths: every pool on the streaming tile kernel
    ("random", 2048, 512, 64, 12, 4),     # wide rows, several steps of 64 columns
    ("random", 96, 32, 50, 8, 3),         # three lane blocks: the second step is half empty; fewer rows than a block
    ("random", 160, 288, 70, 6, 2),       # five lane blocks; rows that spill into a second row block
    ("pack", 512, 128, 700, 4, 2),        # about 350 pairs per expert: several tiles of 128 pairs each
    ("random", 256, 64, 1500, 16, 4),     # 6000 pairs: the route plan places them with its second, multi-block kernel
])
def test_prefill_shapes_vs_oracle(mode, hidden, inter, tokens, experts, k):
    import torch
    from mfq_amd import runtime as R
    import synth
    tensors, runtimes, _ = _layer(f"test/moe/prefill/{mode}/{hidden}/{inter}/{experts}", experts, hidden, inter, mode)
    x = synth.to_bf16(synth.normal(f"test/prefill/shapes/x/{tokens}/{hidden}", (tokens, hidden)))
    ids = synth.zipf_routes(f"test/prefill/shapes/ids/{tokens}/{experts}", tokens, experts, k)
    weights = np.full((tokens, k), 1.0 / k, dtype=np.float32)
    args = (torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda())
    expect = oracle_layer(x, ids, weights, tensors)
    tiles = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=tokens, launch_mode=0).run(*args).cpu().numpy()
    exact = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=tokens, launch_mode=1).run(*args).cpu().numpy()
    err, err_exact = rel_l2(tiles, expect), rel_l2(exact, expect)
    print(f"prefill {mode} H={hidden} I={inter} T={tokens}: streaming {err:.3e} exact {err_exact:.3e}")
    assert err <= FFN_TOL and err_exact <= FFN_TOL


@pytest.mark.parametrize("uniform", ["NINT2", "NINT3", "NINT4", "NINT8", "NVQ3J-L", "MXFP4"])
def test_prefill_uniform_layer(uniform):
    """Every weight class of the streaming tile kernel on its own, quantised weights with one code width."""
    import torch
    from mfq_amd import runtime as R
    import synth
    experts, hidden, inter, k, tokens = 6, 512, 128, 3, 150
    tensors, runtimes, _ = _layer(f"test/moe/prefill/uniform/{uniform}", experts, hidden, inter, "pack", uniform=uniform)
    x = synth.to_bf16(synth.normal("test/prefill/uniform/x", (tokens, hidden)))
    ids = synth.zipf_routes("test/prefill/uniform/ids", tokens, experts, k)
    weights = np.full((tokens, k), 1.0 / k, dtype=np.float32)
    out = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=tokens).run(
        torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda()).cpu().numpy()
    err = rel_l2(out, oracle_layer(x, ids, weights, tensors))
    print(f"prefill uniform {uniform}: rel-L2 {err:.3e}")
    assert err <= FFN_TOL


@pytest.mark.parametrize("uniform", ["NINT2", "NINT3", "NINT4", "NVQ3J-L", "MXFP4"])
def test_prefill_rows_longer_than_a_window(uniform):
    """4096 and 3072 columns are 64 and 48 steps of the tile kernel: more than one window of group levels (NINT),
    block scales (MXFP4) or sign masks and states (NVQ) holds, at either tile height, so the windows move inside a
    block.  Zipf routing over six experts gives tiles of every height: the popular experts fill tiles of 128 pairs,
    the others stay at or below 64, where the windows are the longer ones.  2144 columns (67 lane blocks) take the
    converting path, whose last step lies in a second window and ends in a lane block behind the end of the row."""
    import torch
    from mfq_amd import runtime as R
    import synth
    experts, inter, k, tokens = 6, 128, 3, 220
    for hidden in (4096, 3072, 2144):
        # quantised weights where the packer is quick; random codes, sign masks and states for NVQ (its search over the
        # codebook takes minutes at this width)
        mode = "random" if uniform.startswith("NVQ") else "pack"
        tensors, runtimes, _ = _layer(f"test/moe/prefill/long/{uniform}/{hidden}", experts, hidden, inter, mode, uniform=uniform)
        x = synth.to_bf16(synth.normal(f"test/prefill/long/x/{hidden}", (tokens, hidden)))
        ids = synth.zipf_routes("test/prefill/long/ids", tokens, experts, k)
        counts = np.bincount(ids.ravel(), minlength=experts)
        assert counts.max() > 128 and 0 < counts.min() <= 64, "the case needs tall and low tiles"
        weights = np.full((tokens, k), 1.0 / k, dtype=np.float32)
        out = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=tokens).run(
            torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda()).cpu().numpy()
        err = rel_l2(out, oracle_layer(x, ids, weights, tensors))
        print(f"prefill {uniform} H={hidden}: pairs per expert {sorted(counts.tolist())} rel-L2 {err:.3e}")
        assert err <= FFN_TOL


def test_prefill_f16_activations_and_stage_buffers():
    """fp16 activations take the pair shuffle without conversion; gate/up and pair outputs match the oracle stages."""
    import torch
    from mfq_amd import runtime as R
    import synth
    experts, hidden, inter, k, tokens = 12, 512, 128, 4, 90
    tensors, runtimes, _ = _layer("test/moe/prefill/f16", experts, hidden, inter, "random")
    x = synth.normal("test/prefill/f16/x", (tokens, hidden)).astype(np.float16)
    ids = synth.zipf_routes("test/prefill/f16/ids", tokens, experts, k)
    weights = np.full((tokens, k), 1.0 / k, dtype=np.float32)
    ffn = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=tokens, x_dtype=torch.float16)
    out = ffn.run(torch.from_numpy(x).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda()).cpu().numpy()
    expect = oracle_layer(x.astype(np.float32), ids, weights, tensors)
    assert rel_l2(out, expect) <= FFN_TOL


def test_prefill_equals_decode_path():
    """Same inputs through both kernel families agree to fp16-tile rounding."""
    import torch
    from mfq_amd import runtime as R
    experts, hidden, inter, k, tokens = 24, 512, 128, 6, 16
    tensors, runtimes, _ = _layer("test/moe/random", experts, hidden, inter, "random")
    x, ids, weights = _inputs("test/moe/both", tokens, experts, hidden, k)
    args = (torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(weights).cuda())
    a = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=16, decode_token_limit=32).run(*args).cpu().numpy()
    b = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=16, decode_token_limit=1).run(*args).cpu().numpy()
    assert rel_l2(b, a) <= FFN_TOL


def test_grouped_matmul_and_container_reader():
    """MixedMoeRuntime::forward equivalent, with the tensor loaded by the C++ MFE container reader."""
    import torch
    from mfq_amd import runtime as R
    import synth
    from mfq_amd.formats.mfe import pack_mfe
    experts, hidden, inter, k = 12, 256, 64, 4
    tensors, _ = synth.build_layer("test/moe/grouped", experts, hidden, inter, mix=ALL_FORMATS, mode="random")
    gate = R.MixedMoeRuntime.from_blob(pack_mfe(tensors[0]))
    ogate = OracleMoeTensor(tensors[0])
    for tokens in (3, 20):
        x = synth.to_bf16(synth.normal(f"test/grouped/x/{tokens}", (tokens, hidden)))
        ids = np.stack([np.random.default_rng(t).permutation(experts)[:k] for t in range(tokens)]).astype(np.int32)
        out = gate.forward(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda()).cpu().numpy()
        for t in range(tokens):
            for r in range(k):
                expect = ogate.projection(int(ids[t, r])).rows(x[t:t + 1])[0]
                assert rel_l2(out[t, r].astype(np.float32), expect) < 2e-3


def test_swiglu_and_reduce_ops():
    import torch
    from mfq_amd import runtime as R
    rng = np.random.default_rng(9)
    g = rng.normal(0, 2, 4096).astype(np.float16)
    u = rng.normal(0, 2, 4096).astype(np.float16)
    # zeros of both signs and products that underflow to a zero: the sign of the zero is part of the bits
    g[:8] = [0.0, -0.0, -6e-8, 6e-8, -1e-7, 3.0, -3.0, -0.0]
    u[:8] = [3.0, 3.0, 2.0, -2.0, 1e-4, -0.0, 0.0, -0.0]
    got = R.swiglu(torch.from_numpy(g).cuda(), torch.from_numpy(u).cuda()).cpu().numpy()
    expect = np.array([O.lib().orc_swiglu_f16(int(a), int(b), 0.0) for a, b in zip(g.view(np.uint16), u.view(np.uint16))],
                      dtype=np.uint16)
    assert np.array_equal(got.view(np.uint16), expect)
    pairs = rng.normal(0, 1, (5, 10, 64)).astype(np.float16)
    w = rng.uniform(0, 1, (5, 10)).astype(np.float32)
    got = R.moe_weighted_reduce(torch.from_numpy(pairs).cuda(), torch.from_numpy(w).cuda()).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), O.weighted_reduce(pairs, w).view(np.uint32))


def test_shared_gate_epilogue_bit_exact():
    import torch
    from mfq_amd import runtime as R
    rng = np.random.default_rng(19)
    for tokens, routes, width in ((1, 8, 2048), (5, 10, 72), (33, 4, 1000), (0, 4, 64)):
        pairs = rng.normal(0, 1, (tokens, routes, width)).astype(np.float16)
        w = rng.uniform(0, 1, (tokens, routes)).astype(np.float32)
        shared = rng.normal(0, 1, (tokens, width)).astype(np.float16)
        gate = rng.normal(0, 4, tokens).astype(np.float32)
        gate[:3] = [0.0, 60.0, -60.0][:min(tokens, 3)]
        dev = [torch.from_numpy(a).cuda() for a in (pairs, w, shared, gate)]
        got = R.moe_weighted_reduce_shared_gate(*dev).cpu().numpy()
        expect = O.weighted_reduce_shared_gate(pairs, w, shared, gate)
        assert np.array_equal(got.view(np.uint16), expect.view(np.uint16)), (tokens, routes, width)
        routed = O.weighted_reduce(pairs, w).astype(np.float16)
        got = R.moe_add_shared_gate(torch.from_numpy(routed).cuda(), dev[2], dev[3]).cpu().numpy()
        assert np.array_equal(got.view(np.uint16), expect.view(np.uint16)), (tokens, routes, width)
