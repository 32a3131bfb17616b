"""The allocation-free grouped projection (static device scratch) against the entry point with a caller workspace:
bit-identical outputs on two calls in a row, the second with a smaller input, through the C ABI."""

import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _run(lib, L, tensor, x, ids, static):
    import torch
    tokens, k = ids.shape
    out = torch.full((tokens, k, tensor.out_per_expert), float("nan"), dtype=torch.float16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    dtype = {torch.bfloat16: L.BF16, torch.float16: L.F16}[x.dtype]
    rows_per_token = 1 if x.dim() == 2 else k
    if static:
        L.check(lib.mfq_amd_grouped_matmul_static(C.byref(tensor.struct), x.data_ptr(), dtype, rows_per_token, ids.data_ptr(),
                                                  tokens, k, out.data_ptr(), stream))
    else:
        nbytes = lib.mfq_amd_grouped_matmul_workspace(tokens, k, tensor.experts)
        workspace = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
        L.check(lib.mfq_amd_grouped_matmul(C.byref(tensor.struct), x.data_ptr(), dtype, rows_per_token, ids.data_ptr(),
                                           tokens, k, out.data_ptr(), workspace.data_ptr(), nbytes, stream))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_static_scratch_entry_point_matches_the_workspace_entry_point():
    import torch
    from mfq_amd import _lib as L, runtime as R
    import synth
    from helpers import OracleMoeTensor, rel_l2
    lib = L.lib()
    L.check(lib.mfq_amd_init())
    assert lib.mfq_amd_grouped_matmul_static_capacity() == 128 * 1024
    experts, hidden, inter, k = 24, 512, 128, 6
    mix = (("NINT2", 1 / 6), ("NINT3", 1 / 6), ("NINT4", 1 / 6), ("NINT8", 1 / 6), ("NVQ3J-L", 1 / 6), ("MXFP4", 1 / 6))
    tensors, _ = synth.build_layer("test/static", experts, hidden, inter, mix=mix, mode="random")
    gate = R.MixedMoeRuntime(tensors[0])
    oracle = OracleMoeTensor(tensors[0])
    # the largest call first (512 tokens = 3072 pairs: the large plan kernel with its dynamic LDS and the tile kernels,
    # near the top of what the static array holds), then smaller ones (40: the small plan and tile kernels, 7 and 1: the
    # decode kernels) that reuse the scratch
    assert 64 * 1024 < lib.mfq_amd_grouped_matmul_workspace(512, k, experts) <= lib.mfq_amd_grouped_matmul_static_capacity()
    for tokens in (512, 40, 7, 40, 1):
        x = synth.to_bf16(synth.normal(f"test/static/x/{tokens}", (tokens, hidden)))
        ids = np.stack([np.random.default_rng(50 + t).permutation(experts)[:k] for t in range(tokens)]).astype(np.int32)
        ids[0, 0] = -1 if tokens > 1 else ids[0, 0]           # an unrouted pair
        xd, idd = torch.from_numpy(x).to(torch.bfloat16).cuda(), torch.from_numpy(ids).cuda()
        want = _run(lib, L, gate, xd, idd, static=False)
        got = _run(lib, L, gate, xd, idd, static=True)
        routed = ids >= 0
        assert np.array_equal(got.view(np.uint16)[routed], want.view(np.uint16)[routed]), tokens
        for t in range(min(tokens, 3)):
            for r in range(k):
                if ids[t, r] >= 0:
                    expect = oracle.projection(int(ids[t, r])).rows(x[t:t + 1])[0]
                    assert rel_l2(got[t, r].astype(np.float32), expect) < 2e-3


def test_static_scratch_entry_point_rejects_what_does_not_fit():
    import torch
    from mfq_amd import _lib as L, runtime as R
    import synth
    lib = L.lib()
    L.check(lib.mfq_amd_init())
    tensors, _ = synth.build_layer("test/static/small", 8, 64, 32, mix=(("NINT4", 1.0),), mode="random")
    gate = R.MixedMoeRuntime(tensors[0])
    tokens, k = 4096, 8                                     # 32768 pairs: the plan lists alone exceed 128 KiB
    assert lib.mfq_amd_grouped_matmul_workspace(tokens, k, 8) > lib.mfq_amd_grouped_matmul_static_capacity()
    x = torch.zeros((tokens, 64), dtype=torch.bfloat16, device="cuda")
    ids = torch.zeros((tokens, k), dtype=torch.int32, device="cuda")
    out = torch.zeros((tokens, k, 32), dtype=torch.float16, device="cuda")
    status = lib.mfq_amd_grouped_matmul_static(C.byref(gate.struct), x.data_ptr(), L.BF16, 1, ids.data_ptr(), tokens, k,
                                               out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert status == L.ERR_INVALID and b"exceeds the static scratch" in lib.mfq_amd_last_error()
