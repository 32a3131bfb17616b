"""The benchmark's own layers at full size (512 experts x (2048 <-> 512), top-10, mixed formats) through the C ABI.

The weights are the random packed pools of tests/benchdata.py, built in device memory; the oracle reads the
experts a check needs back from the device (runtime layout, one expert at a time), so the CPU side stays at a few
seconds.  Checks: the decode batch against the oracle end to end (ids bit-exact, output rel-L2 <= 1e-3), sampled
tokens of the 4096-token prefill against the oracle, and two properties that do not depend on size: doubling the
route weights doubles the output bit for bit, and permuting the tokens of a batch permutes the outputs bit for bit.
"""

import numpy as np
import pytest

from helpers import rel_l2
from oracle import oracle as O

pytestmark = pytest.mark.gpu

FFN_TOL = 1e-3
EXPERTS, HIDDEN, INTER, TOP_K = 512, 2048, 512, 10

_STATE = {}


def _layer():
    """One full-size mixed-format layer, shared by the tests of this file."""
    if "layer" not in _STATE:
        import benchdata
        import synth
        formats = [synth.draw_formats(f"cfg4/format/{p}", EXPERTS) for p in ("gate", "up", "down")]
        _STATE["layer"] = benchdata.device_layer("test/full/layer", EXPERTS, HIDDEN, INTER, formats)
    return _STATE["layer"]


def _oracle_projections(layer):
    cache = {}

    def of(expert):
        if expert not in cache:
            cache[expert] = tuple(O.Projection(t.host_layout(expert)) for t in layer)
        return cache[expert]
    return of


def _decode_inputs(tokens):
    import torch
    from mfq_amd import runtime as R
    import synth
    x = synth.to_bf16(synth.normal(f"test/full/x/{tokens}", (tokens, HIDDEN)))
    router = synth.to_bf16(synth.normal("test/full/router", (EXPERTS, HIDDEN), 0.02))
    xd = torch.from_numpy(x).to(torch.bfloat16).cuda()
    logits = R.router_logits(xd, torch.from_numpy(router).to(torch.bfloat16).cuda())
    return x, router, xd, logits


@pytest.mark.parametrize("tokens", [1, 4, 16])      # one wave per token in the plan's top-k up to 8 tokens, half a wave above
def test_decode_batch_vs_oracle(tokens):
    from mfq_amd import runtime as R
    layer = _layer()
    x, router, xd, logits = _decode_inputs(tokens)
    ffn = R.MfeFfnRuntime(*layer, top_k=TOP_K, max_tokens=tokens)
    out = ffn.run_logits(xd, logits).cpu().numpy()
    ids, weights = (t.numpy() for t in ffn.routes(tokens))
    ids_ref, weights_ref = O.topk(O.router_logits(x, router), TOP_K)
    assert np.array_equal(ids, ids_ref)
    assert np.allclose(weights, weights_ref, rtol=1e-6, atol=0)
    expect = O.moe_layer(x, ids_ref, weights_ref, _oracle_projections(layer))
    assert rel_l2(out, expect) <= FFN_TOL


def test_prefill_4096_sampled_tokens_vs_oracle():
    import torch
    from mfq_amd import runtime as R
    import synth
    layer = _layer()
    tokens = 4096
    x = synth.to_bf16(synth.normal("test/full/prefill/x", (tokens, HIDDEN)))
    ids = synth.zipf_routes("test/full/prefill/zipf", tokens, EXPERTS, TOP_K)
    weights = np.random.default_rng(5).uniform(0.02, 0.3, (tokens, TOP_K)).astype(np.float32)
    ffn = R.MfeFfnRuntime(*layer, top_k=TOP_K, max_tokens=tokens)
    out = ffn.run(torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda(),
                  torch.from_numpy(weights).cuda()).cpu().numpy()
    assert np.isfinite(out).all()
    # tokens spread over the batch, among them one routed to the most popular expert (tiles of 128 pairs)
    # and the last token
    counts = np.bincount(ids.ravel(), minlength=EXPERTS)
    busiest = int(np.argmax(counts))
    sample = sorted({0, 1, 777, 2048, 4095, int(np.argwhere((ids == busiest).any(axis=1))[0, 0])})
    expect = O.moe_layer(x[sample], ids[sample], weights[sample], _oracle_projections(layer))
    assert rel_l2(out[sample], expect) <= FFN_TOL
    for row, want in zip(out[sample], expect):
        assert rel_l2(row, want) <= 2 * FFN_TOL


def test_doubling_route_weights_doubles_the_output_exactly():
    import torch
    from mfq_amd import runtime as R
    layer = _layer()
    for tokens in (4, 200):                                   # the decode kernels and the tile kernels
        x, _, xd, logits = _decode_inputs(tokens)
        ids, weights = R.moe_topk(logits, TOP_K)
        ffn = R.MfeFfnRuntime(*layer, top_k=TOP_K, max_tokens=tokens)
        once = ffn.run(xd, ids, weights).cpu().numpy()
        twice = ffn.run(xd, ids, weights * 2.0).cpu().numpy()
        assert np.array_equal((2.0 * once).view(np.uint32), twice.view(np.uint32))
        assert np.abs(once).max() > 0


def test_permuting_the_tokens_permutes_the_outputs_exactly():
    import torch
    from mfq_amd import runtime as R
    layer = _layer()
    tokens = 16
    x, _, xd, logits = _decode_inputs(tokens)
    ids, weights = R.moe_topk(logits, TOP_K)
    ffn = R.MfeFfnRuntime(*layer, top_k=TOP_K, max_tokens=tokens)
    base = ffn.run(xd, ids, weights).cpu().numpy()
    order = torch.from_numpy(np.random.default_rng(9).permutation(tokens)).cuda()
    moved = ffn.run(xd[order].contiguous(), ids[order].contiguous(), weights[order].contiguous()).cpu().numpy()
    assert np.array_equal(moved.view(np.uint32), base[order.cpu().numpy()].view(np.uint32))
