"""The grouped GEMM kernels run on the CPU: csrc/grouped_gemm.hip itself, compiled for the host, under an emulation of a
gfx950 workgroup (tests/host/gemm_emulation.cpp, tests/host/shim/hip/hip_runtime.h - one coroutine per lane, the matrix
instruction, the transposing LDS read and the direct global -> LDS copy modelled by their lane layouts).  Both loops
of the kernel, eight and four wavefronts per tile, go through the C entry points on problems whose sums are exact in
fp32, so every output must equal the reference product bit for bit; every address a copy reads is checked against its
operand; and the copies land either at once or as late as the kernel's own waits allow.  The eight-wave loop's results
on the GPU are pinned by the GPU tests, which makes it the check of the emulation; the four-wave loop then has to pass
the same cases.  A run with every wait eight copies short must fail: the checker sees a broken protocol."""

import os
import shutil
import subprocess

import pytest


HOST_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host")


def _host_clang():
    # the kernel source uses clang's vector extensions and __bf16: the host compiler is the ROCm toolchain's clang
    for candidate in (shutil.which("amdclang++"), "/opt/rocm/llvm/bin/clang++", "/opt/rocm/bin/amdclang++"):
        if candidate and os.path.exists(candidate):
            return candidate
    return None


@pytest.fixture(scope="module")
def emulation(tmp_path_factory):
    compiler = _host_clang()
    if compiler is None:
        pytest.skip("no clang of the ROCm toolchain to build the host emulation with")
    binary = str(tmp_path_factory.mktemp("gemm_emulation") / "gemm_emulation")
    # -O0: the unoptimised build compiles in seconds and, with 512 coroutines switching at every wave-wide instruction,
    # also runs faster than the optimised one
    subprocess.run([compiler, "-std=c++17", "-O0", "-I", os.path.join(HOST_DIR, "shim"), "-Wno-unknown-attributes",
                    "-Wno-ignored-attributes", "-Wno-unused-value", "-Wno-psabi", os.path.join(HOST_DIR, "gemm_emulation.cpp"),
                    "-o", binary], check=True)
    return binary


@pytest.mark.parametrize("waves", ["8", "4"])
def test_grouped_gemm_loops_under_emulation(emulation, waves):
    result = subprocess.run([emulation, waves], capture_output=True, text=True, timeout=900)
    assert result.returncode == 0, result.stdout + result.stderr
    assert result.stdout.startswith("ok: 15 cases"), result.stdout


@pytest.mark.parametrize("waves", ["8", "4"])
def test_the_emulation_notices_waits_that_are_too_short(emulation, waves):
    result = subprocess.run([emulation, waves, "--lax-waits"], capture_output=True, text=True, timeout=900)
    assert result.returncode == 1 and "FAILED" in result.stdout and "expected" in result.stdout, result.stdout + result.stderr
