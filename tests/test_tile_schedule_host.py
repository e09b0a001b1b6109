"""The tile scheduling of the grouped GEMM (csrc/ck_tile_schedule.h: which expert, row tile, column tile and piece of
the contraction a workgroup takes) is device code that runs before any bounds could be checked on the device.  Its
source compiles for the host as well, with a wavefront emulated lane by lane (tests/host/tile_schedule_host.cpp), and
there every workgroup of every launch form is walked for expert_offsets of many shapes - balanced and skewed loads,
empty experts, one row in total, more than 64 experts, one to 112 column tiles, contractions with and without a tail
to split: every tile exactly once, rows inside their expert, pieces of a split tile covering the contraction exactly,
slots inside the workspace, the fix-up launch matching the first, weight-gradient tiles in the order of falling load."""

import os
import shutil
import subprocess

import pytest


HOST_SOURCE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host", "tile_schedule_host.cpp")


@pytest.fixture(scope="module")
def harness(tmp_path_factory):
    compiler = shutil.which("g++")
    if compiler is None:
        pytest.skip("no host C++ compiler")
    binary = str(tmp_path_factory.mktemp("tile_schedule") / "tile_schedule_host")
    subprocess.run([compiler, "-O2", "-std=c++17", "-Wall", HOST_SOURCE, "-o", binary], check=True)
    return binary


def test_every_tile_is_dealt_exactly_once(harness):
    result = subprocess.run([harness], capture_output=True, text=True, timeout=600)
    assert result.returncode == 0, result.stdout + result.stderr
    assert result.stdout.startswith("ok:"), result.stdout


def test_the_harness_notices_a_grid_that_is_too_short(harness):
    result = subprocess.run([harness, "--short-grid"], capture_output=True, text=True, timeout=600)
    assert result.returncode == 1 and "tiles missing" in result.stdout, result.stdout + result.stderr
