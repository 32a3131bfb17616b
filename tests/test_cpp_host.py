"""The C ABI from the reference's own host language: include/mfq_amd.h must be valid C and C++, and the C++
classes of include/mfq_amd.hpp (MixedMoeRuntime, MfeFfnRuntime, moe_topk) must give, from a program with no
Python and no torch in it (tests/cpp/host_mirror_check, built by ``python -m mfq_amd.build``), what the oracle
gives and bit for bit what the Python mirror gives on the same containers and inputs."""

import subprocess
from pathlib import Path

import numpy as np
import pytest

from helpers import oracle_layer, rel_l2
import synth
from mfq_amd.formats import mfe as MFE, mx, nint, nvq
from mfq_amd.quantize import nint_quant, nvq_quant
from oracle import oracle as O

ROOT = Path(__file__).resolve().parent.parent
PROGRAM = ROOT / "tests" / "cpp" / "host_mirror_check"
ALL_FORMATS = (("NINT2", 1 / 6), ("NINT3", 1 / 6), ("NINT4", 1 / 6), ("NINT8", 1 / 6), ("NVQ3J-L", 1 / 6), ("MXFP4", 1 / 6))


def _program():
    assert PROGRAM.exists(), f"{PROGRAM} is missing: run `python -m mfq_amd.build`"
    return str(PROGRAM)


def test_headers_compile_as_c_and_as_cpp(tmp_path):
    c_unit = tmp_path / "unit.c"
    c_unit.write_text('#include "mfq_amd.h"\nint main(void) { mfq_amd_projection p; (void)p; return mfq_amd_abi_version() < 0; }\n')
    done = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", f"-I{ROOT / 'include'}",
                           "-fsyntax-only", str(c_unit)], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
    cpp_unit = tmp_path / "unit.cpp"
    cpp_unit.write_text('#include "mfq_amd.hpp"\nint main() { mfq_amd::MfeFfnOptions o; return o.top_k - 1; }\n')
    done = subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", f"-I{ROOT / 'include'}", "-fsyntax-only",
                           str(cpp_unit)], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr


def test_cpp_reads_a_container_and_reports_malformed_ones(tmp_path):
    rng = np.random.default_rng(31)
    out, width = 4, 96
    pools = [
        MFE.MfePool(np.array([2, 0], dtype=np.int32), nint_quant.random_codes(2 * out, width, nint.NintSpec(4, 24, 6), rng)),
        MFE.MfePool(np.array([1], dtype=np.int32), nvq_quant.random_nvq_jsc(out, width, nvq.NVQ3_D4_1024, rng)),
        MFE.MfePool(np.array([3], dtype=np.int32), mx.random_mxfp4(out, width, rng)),
    ]
    blob = MFE.pack_mfe(MFE.MfeTensor((4, out, width), pools))
    good = tmp_path / "good.mfe"
    good.write_bytes(blob)
    done = subprocess.run([_program(), "parse", str(good)], capture_output=True, text=True)
    assert done.returncode == 0, done.stdout + done.stderr
    assert done.stdout.split("\n")[:4] == ["4 4 96 3", "2 0", "1", "3"]
    bad = tmp_path / "bad.mfe"
    bad.write_bytes(blob[:-5])
    done = subprocess.run([_program(), "parse", str(bad)], capture_output=True, text=True)
    assert done.returncode == 3 and done.stdout.startswith("error: ") and "truncated" in done.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("tokens", [3, 40])                 # the decode kernels and the tile kernels
def test_cpp_ffn_equals_the_python_mirror_and_the_oracle(tmp_path, tokens):
    import torch
    from mfq_amd import runtime as R
    experts, hidden, inter, k = 16, 512, 128, 4
    tensors, _ = synth.build_layer("test/cpp/layer", experts, hidden, inter, mix=ALL_FORMATS, mode="random")
    blobs = [MFE.pack_mfe(t) for t in tensors]
    for name, blob in zip(("gate", "up", "down"), blobs):
        (tmp_path / f"{name}.mfe").write_bytes(blob)
    x = synth.to_bf16(synth.normal(f"test/cpp/x/{tokens}", (tokens, hidden)))
    router = synth.to_bf16(synth.normal("test/cpp/router", (experts, hidden), 0.02))
    xd = torch.from_numpy(x).to(torch.bfloat16).cuda()
    logits = R.router_logits(xd, torch.from_numpy(router).to(torch.bfloat16).cuda())
    (tmp_path / "x.bf16").write_bytes(xd.cpu().view(torch.int16).numpy().tobytes())
    (tmp_path / "logits.f32").write_bytes(logits.cpu().numpy().astype(np.float32).tobytes())

    print(f"host_mirror_check ffn tokens={tokens}", flush=True)
    done = subprocess.run([_program(), "ffn", str(tmp_path), str(tokens), str(k), str(experts), str(hidden)],
                          capture_output=True, text=True, timeout=120)
    assert done.returncode == 0 and done.stdout.strip().endswith("ok"), done.stdout + done.stderr

    def read(name, dtype, shape):
        return np.frombuffer((tmp_path / name).read_bytes(), dtype=dtype).reshape(shape)

    ids, weights = read("ids.i32", np.int32, (tokens, k)), read("weights.f32", np.float32, (tokens, k))
    fused, separate = read("out_logits.f32", np.float32, (tokens, hidden)), read("out_routes.f32", np.float32, (tokens, hidden))
    ids_ref, weights_ref = O.topk(O.router_logits(x, router), k)
    assert np.array_equal(ids, ids_ref)
    assert np.allclose(weights, weights_ref, rtol=1e-6, atol=0)
    assert np.array_equal(fused.view(np.uint32), separate.view(np.uint32))
    assert rel_l2(fused, oracle_layer(x, ids_ref, weights_ref, tensors)) <= 1e-3
    # the Python mirror on the same containers
    runtimes = [R.MixedMoeRuntime.from_blob(blob) for blob in blobs]
    mirror = R.MfeFfnRuntime(*runtimes, top_k=k, max_tokens=tokens).run_logits(xd, logits).cpu().numpy()
    assert np.array_equal(fused.view(np.uint32), mirror.view(np.uint32))


def test_streaming_fetches_stay_inside_their_fields(tmp_path):
    """The address arithmetic the streaming kernels run on the device (mfq_amd/csrc/fetch_at.h), compiled for the host
    and swept over every kernel class, widths from 32 to 4096, 1..70 rows and up to three experts per pool: no fetch
    reads a byte outside the packed field it reads from (including the NVQ sign-mask load, which is not clamped)."""
    import shutil
    import subprocess
    compiler = shutil.which("g++") or shutil.which("hipcc")
    if compiler is None:
        pytest.skip("no host C++ compiler")
    binary = tmp_path / "fetch_extent_check"
    source = ROOT / "tests" / "cpp" / "fetch_extent_check.cpp"
    subprocess.run([compiler, "-O2", "-std=c++17", str(source), "-o", str(binary)], check=True)
    done = subprocess.run([str(binary)], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
    assert "fetches inside their fields" in done.stdout and int(done.stdout.split()[0]) > 1_000_000


def test_tile_kernel_windows_hold_what_the_steps_read(tmp_path):
    """The LDS windows of the prefill tile kernel (mfq_amd/csrc/tile_windows.h), compiled for the host and swept over
    widths from 64 to 8192, both window lengths, every group size and side windows of up to 8 and 16 steps: every level,
    block scale, sign mask and state a step reads lies in what its window staged, and the decode one step ahead stays
    inside the row's own piece of LDS."""
    import shutil
    import subprocess
    compiler = shutil.which("g++") or shutil.which("hipcc")
    if compiler is None:
        pytest.skip("no host C++ compiler")
    binary = tmp_path / "tile_window_check"
    subprocess.run([compiler, "-O2", "-std=c++17", str(ROOT / "tests" / "cpp" / "tile_window_check.cpp"), "-o", str(binary)], check=True)
    done = subprocess.run([str(binary)], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
    assert "window reads inside what was staged" in done.stdout and int(done.stdout.split()[0]) > 10_000_000


def test_e4m3_split_rounding_and_scales(tmp_path):
    """mfq_amd/csrc/fp8_split.h compiled for the host: E4M3 rounding against all byte values (nearest, ties to even,
    saturation), the E8M0 block scale rule, and hi + lo adding up to bf16 sources."""
    import shutil
    import subprocess
    compiler = shutil.which("g++") or shutil.which("hipcc")
    if compiler is None:
        pytest.skip("no host C++ compiler")
    binary = tmp_path / "fp8_split_check"
    subprocess.run([compiler, "-O2", "-std=c++17", str(ROOT / "tests" / "cpp" / "fp8_split_check.cpp"), "-o", str(binary)], check=True)
    done = subprocess.run([str(binary)], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr
    assert "roundings checked" in done.stdout
