"""Host code under AddressSanitizer and UBSan (no GPU needed).

1. The packed block format's index arithmetic (csrc/tq_layout.h, the header the kernels include) is compiled
   for the host and run against exactly sized heap buffers on blocks the oracle packed: reads, writes and
   offsets that leave their block would be reported.
2. The C ABI's argument checks (csrc/capi.hip, host pass compiled with the sanitizers) are driven with null
   pointers, negative sizes, bad enums and misaligned pointers.
"""
import os
import shutil
import subprocess

import numpy as np
import pytest

import tq_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "turboquant_plus_amd", "csrc")
HERE = os.path.join(ROOT, "tests", "host_check")
SAN = ["-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer", "-g", "-O1"]
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
ENV.pop("LD_PRELOAD", None)     # the sanitizer runtime must come first in the library list of these two programs


@pytest.fixture(scope="module")
def layout_check(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("host_check") / "layout_check")
    subprocess.run(["g++", "-std=c++17", *SAN, "-I", CSRC, os.path.join(HERE, "layout_check.cpp"), "-o", exe], check=True)
    return exe


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("kind", ["k", "v"])
@pytest.mark.parametrize("tokens", [128, 384])
def test_layout_arithmetic_under_sanitizers(layout_check, tmp_path, bits, kind, tokens):
    rng = np.random.default_rng(bits * 100 + tokens + (kind == "v"))
    idx = rng.integers(0, 1 << bits, size=(tokens, 128)).astype(np.uint8)
    g = rng.standard_normal(tokens).astype(np.float16)
    packed = O.layout_pack(idx, g, bits, kind)
    path = tmp_path / "case.bin"
    with open(path, "wb") as f:
        f.write(np.array([bits, 0 if kind == "k" else 1, tokens], dtype=np.int32).tobytes())
        f.write(idx.tobytes())
        f.write(g.view(np.uint16).tobytes())
        f.write(np.ascontiguousarray(packed).tobytes())
    r = subprocess.run([layout_check, str(path)], capture_output=True, text=True, env=ENV)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "layout ok" in r.stdout


def test_launch_constant_divider(layout_check):
    """tqd::FastDiv (the kernels' division by the blocks per sequence) equals the plain division."""
    r = subprocess.run([layout_check, "fastdiv"], capture_output=True, text=True, env=ENV)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "fastdiv ok" in r.stdout


def test_abi_argument_paths_under_sanitizers(tmp_path):
    hipcc = shutil.which("hipcc")
    if hipcc is None:
        pytest.skip("hipcc not on PATH")
    objs = [os.path.join(CSRC, "build", n + ".o") for n in ("api_kernels", "turbo_kernels", "attn_kernels")]
    if not all(os.path.exists(o) for o in objs):
        pytest.skip("kernel objects not built (make -C turboquant_plus_amd/csrc)")
    host_san = []
    for flag in ("-fsanitize=address", "-fsanitize=undefined", "-fno-sanitize-recover=all"):
        host_san += ["-Xarch_host", flag]
    common = [hipcc, "--offload-arch=gfx950", "-std=c++17", "-O1", "-g", "-I", os.path.join(ROOT, "include"), "-I", CSRC,
              "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument"]
    capi_o, main_o, exe = str(tmp_path / "capi_san.o"), str(tmp_path / "abi_args.o"), str(tmp_path / "abi_args")
    subprocess.run(common + host_san + ["-c", os.path.join(CSRC, "capi.hip"), "-o", capi_o], check=True,
                   stderr=subprocess.DEVNULL)
    subprocess.run(common + host_san + ["-x", "hip", "-c", os.path.join(HERE, "abi_args.cpp"), "-o", main_o], check=True,
                   stderr=subprocess.DEVNULL)
    subprocess.run([hipcc, "--offload-arch=gfx950", "-fsanitize=address", "-fsanitize=undefined", "-fno-gpu-sanitize",
                    main_o, capi_o, *objs, "-o", exe], check=True, stderr=subprocess.DEVNULL)
    r = subprocess.run([exe], capture_output=True, text=True, env=ENV)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "abi argument paths ok" in r.stdout
