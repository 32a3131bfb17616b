"""GPU parity of routing through the C ABI: logits bit-exact, top-k ids bit-exact, route
weights within a few ulp, route plan identical to the oracle (= bincount / cumsum)."""

import numpy as np
import pytest

from helpers import bits_equal
from oracle import oracle as O

pytestmark = pytest.mark.gpu


def _router_case(tokens, experts, width, seed):
    import synth
    x = synth.to_bf16(synth.normal(f"test/route/x/{seed}", (tokens, width)))
    router = synth.to_bf16(synth.normal(f"test/route/w/{seed}", (experts, width), 0.02))
    return x, router


@pytest.mark.parametrize("tokens,experts,width", [(1, 512, 2048), (16, 512, 2048), (5, 40, 100), (3, 1000, 64)])
def test_router_logits_bit_exact(tokens, experts, width):
    import torch
    from mfq_amd import runtime as R
    x, router = _router_case(tokens, experts, width, 1)
    expect = O.router_logits(x, router)
    got = R.router_logits(torch.from_numpy(x).to(torch.bfloat16).cuda(),
                          torch.from_numpy(router).to(torch.bfloat16).cuda()).cpu().numpy()
    assert bits_equal(got, expect)


@pytest.mark.parametrize("tokens,experts,k", [(1, 512, 10), (4, 512, 10), (16, 512, 10), (64, 512, 10),
                                                (7, 40, 4), (3, 1000, 32), (2, 8, 8), (5, 33, 1), (9, 128, 8), (6, 200, 10), (32, 256, 6)])
def test_topk_ids_bit_exact(tokens, experts, k):
    import torch
    from mfq_amd import runtime as R
    x, router = _router_case(tokens, experts, 256, 2)
    logits = O.router_logits(x, router)
    ids_ref, w_ref = O.topk(logits, k)
    ids, w = R.moe_topk(torch.from_numpy(logits).cuda(), k)
    assert np.array_equal(ids.cpu().numpy(), ids_ref)
    np.testing.assert_allclose(w.cpu().numpy(), w_ref, rtol=1e-6, atol=0)
    # the reference's own check: ids equal softmax().topk() (tests/test_moe_kernels_cuda.py:294-300)
    torch_ids = torch.softmax(torch.from_numpy(logits).double(), dim=-1).topk(k, dim=-1).indices.numpy()
    assert np.array_equal(ids.cpu().numpy(), torch_ids)


def test_topk_ties_go_to_lower_id_and_nan_is_lowest():
    import torch
    from mfq_amd import runtime as R
    logits = np.zeros((3, 512), dtype=np.float32)
    logits[1, 100:110] = 1.0
    logits[2, :] = np.linspace(-1, 1, 512)
    logits[2, 511] = np.nan
    ids, w = R.moe_topk(torch.from_numpy(logits).cuda(), 10)
    ids = ids.cpu().numpy()
    assert list(ids[0]) == list(range(10))
    assert list(ids[1]) == list(range(100, 110))
    assert list(ids[2]) == list(range(510, 500, -1))
    ids_ref, w_ref = O.topk(logits, 10)
    assert np.array_equal(ids, ids_ref)
    np.testing.assert_allclose(w.cpu().numpy(), w_ref, rtol=1e-6)
    np.testing.assert_allclose(w.cpu().numpy().sum(-1), 1.0, rtol=1e-5)


def test_topk_half_logits_and_scale():
    import torch
    from mfq_amd import runtime as R
    rng = np.random.default_rng(4)
    logits = rng.normal(0, 2, (6, 512)).astype(np.float16)
    ids, w = R.moe_topk(torch.from_numpy(logits).cuda(), 10, scale=2.5)
    ids_ref, w_ref = O.topk(logits.astype(np.float32), 10, scale=2.5)
    assert np.array_equal(ids.cpu().numpy(), ids_ref)
    np.testing.assert_allclose(w.cpu().numpy(), w_ref, rtol=1e-6)


@pytest.mark.parametrize("tokens,experts,k,tile_m", [(1, 512, 10, 8), (16, 512, 10, 8), (4096, 512, 10, 64),
                                                      (37, 8, 3, 16), (300, 1000, 6, 8), (32, 64, 32, 8), (102, 512, 10, 8), (103, 512, 10, 8)])
def test_route_plan_matches_oracle(tokens, experts, k, tile_m):
    import torch
    from mfq_amd import runtime as R
    import synth
    if tokens >= 4096:
        ids = synth.zipf_routes("test/plan/zipf", tokens, experts, k)
    else:
        ids = np.stack([np.random.default_rng(t).permutation(experts)[:k] for t in range(tokens)]).astype(np.int32)
    plan = R.build_moe_route_plan(torch.from_numpy(ids).cuda(), experts, tile_m)
    ref = O.route_plan(ids, experts, tile_m)
    counts = np.bincount(ids.reshape(-1), minlength=experts)
    assert np.array_equal(plan["counts"].cpu().numpy(), counts)
    assert np.array_equal(plan["expert_bounds"].cpu().numpy(), np.concatenate([[0], np.cumsum(counts)]))
    assert np.array_equal(plan["counts"].cpu().numpy(), ref["counts"])
    assert np.array_equal(plan["tile_bounds"].cpu().numpy(), ref["tile_bounds"])
    ntiles = int(ref["tile_bounds"][-1])
    assert np.array_equal(plan["tile_experts"].cpu().numpy()[:ntiles], ref["tile_experts"])
    assert np.array_equal(plan["ids_dst"].cpu().numpy()[: tokens * k], ref["ids_dst"])


def test_route_plan_skips_invalid_ids():
    import torch
    from mfq_amd import runtime as R
    ids = np.array([[0, 5, -1], [7, 8, 2], [5, 5, 99]], dtype=np.int32)
    plan = R.build_moe_route_plan(torch.from_numpy(ids).cuda(), 8, 8)
    ref = O.route_plan(ids, 8, 8)
    assert np.array_equal(plan["counts"].cpu().numpy(), ref["counts"])
    assert np.array_equal(plan["ids_dst"].cpu().numpy()[: ref["ids_dst"].size], ref["ids_dst"])


def _check_topk(logits, k, **kwargs):
    import torch
    from mfq_amd import runtime as R
    ids_ref, w_ref = O.topk(logits, k, **kwargs)
    ids, w = R.moe_topk(torch.from_numpy(logits).cuda(), k, **kwargs)
    assert np.array_equal(ids.cpu().numpy(), ids_ref)
    np.testing.assert_allclose(w.cpu().numpy(), w_ref, rtol=1e-6, atol=1e-38)


def test_topk_adversarial_layouts():
    """Inputs chosen against the selection's shortcuts: more equal maxima than routes; the large logits crowded into
    one lane's entries (experts 3, 35, 67, ...); logits one unit in the last place apart (numerators that may share a
    probability); a one-hot row (probabilities near the bottom of the range); coarse logits with many exact ties."""
    rng = np.random.default_rng(123)
    rows = []
    a = rng.normal(0, 1, 512).astype(np.float32); a[[5, 37, 69, 100, 101, 200, 300, 301, 302, 400, 450, 511]] = 4.0
    rows.append(a)                                                      # 12 equal maxima, top-10
    b = rng.normal(0, 1, 512).astype(np.float32); b[3::32] = 3.0 + np.arange(16, dtype=np.float32) * 0.125
    rows.append(b)                                                      # the 16 largest in the entries of lane 3
    c = np.float32(1.0) + np.arange(512, dtype=np.float32) * np.float32(2.0 ** -23)
    rows.append(c[::-1].copy())                                         # neighbours one ulp apart, descending by id
    rows.append(c.copy())
    d = np.zeros(512, dtype=np.float32); d[77] = 100.0
    rows.append(d)                                                      # one-hot: the rest underflows to equal tiny values
    e = np.zeros(512, dtype=np.float32); e[77] = 60.0; e[100:140] = rng.normal(0, 0.001, 40)
    rows.append(e)
    rows.append(np.round(rng.normal(0, 1, 512) * 4).astype(np.float32) / 4)     # quantised: many exact ties
    rows.append(np.round(rng.normal(0, 1, 512) * 2).astype(np.float32) / 2)
    rows.append(np.full(512, -1e30, dtype=np.float32))
    f = rng.normal(0, 1, 512).astype(np.float32); f[::3] = np.nan
    rows.append(f)
    logits = np.stack(rows)
    for k in (1, 4, 10, 32):
        _check_topk(logits, k)
    _check_topk(logits, 10, normalize=False, scale=0.5)
    for experts, k in ((40, 4), (33, 8), (64, 32), (1000, 10), (129, 6)):
        sub = np.round(rng.normal(0, 1, (9, experts)) * 3).astype(np.float32) / 3
        _check_topk(sub, k)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_topk_many_random_rows(seed):
    rng = np.random.default_rng(1000 + seed)
    logits = rng.normal(0, [0.02, 1.0, 8.0][seed], (257, 512)).astype(np.float32)
    _check_topk(logits, 10)
    _check_topk(logits[:33, :256].copy(), 8)


@pytest.mark.parametrize("x_dtype,r_dtype", [("f16", "f16"), ("bf16", "f16"), ("f32", "bf16"), ("f32", "f32")])
def test_router_logits_every_operand_type(x_dtype, r_dtype):
    """16-bit operands take the kernel with one thread per logit (fused multiply-add of an exact product), float32
    operands the kernel with separate multiply and add; both give the oracle's sums bit for bit."""
    import torch
    from mfq_amd import runtime as R
    rng = np.random.default_rng(77)
    types = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}
    for tokens, experts, width in ((3, 300, 512), (2, 64, 72), (1, 7, 33)):
        x = torch.from_numpy(rng.normal(0, 1, (tokens, width)).astype(np.float32)).to(types[x_dtype])
        router = torch.from_numpy(rng.normal(0, 0.05, (experts, width)).astype(np.float32)).to(types[r_dtype])
        expect = O.router_logits(x.float().numpy(), router.float().numpy())
        got = R.router_logits(x.cuda(), router.cuda()).cpu().numpy()
        assert bits_equal(got, expect), (x_dtype, r_dtype, tokens, experts, width)
