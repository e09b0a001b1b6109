"""Builds ``lib/libcute_hip.so`` from the HIP sources in ``../csrc`` with hipcc for gfx950.

One shared library, plain C ABI (declared in ``include/cute_hip.h`` at the repository root).  The
reference compiles its CUDA sources lazily, per op, through ``torch.utils.cpp_extension.load``
(cute_kernels/jit.py:16-49); here everything is compiled ahead of time in one step so that the built
library can be shipped next to the Python package.
"""

from __future__ import annotations

import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor


PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC_DIR = os.path.normpath(os.path.join(PACKAGE_DIR, "..", "csrc"))
LIB_DIR = os.path.join(PACKAGE_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libcute_hip.so")

SOURCES = ["status.hip", "add.hip", "swiglu.hip", "rmsnorm.hip", "embedding.hip", "moe_sort.hip", "moe_combine.hip", "expert_bias.hip", "router.hip", "grouped_gemm.hip"]

# -packed-fp32-ops off: the packed fp32 VALU forms are not wanted in any kernel of this library
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


def find_hipcc() -> str:
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise RuntimeError("hipcc not found: the HIP kernels of cute_kernels cannot be built")
    return hipcc


def _compile(hipcc: str, source: str, obj_dir: str, verbose: bool) -> str:
    obj = os.path.join(obj_dir, os.path.splitext(source)[0] + ".o")
    cmd = [hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC_DIR, source), "-o", obj]
    result = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; that line is noise
    stderr = "\n".join(line for line in result.stderr.splitlines() if "packed-fp32-ops" not in line)
    if result.returncode != 0:
        raise RuntimeError(f"hipcc failed on {source}:\n{stderr}")
    if verbose and stderr.strip():
        print(stderr)
    return obj


def build(verbose: bool = False, jobs: int | None = None) -> str:
    """Compile every source and link the shared library; returns its path."""
    hipcc = find_hipcc()
    obj_dir = os.path.join(PACKAGE_DIR, "..", "build", "obj")
    os.makedirs(obj_dir, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    jobs = jobs or min(len(SOURCES), os.cpu_count() or 1, 16)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objects = list(pool.map(lambda src: _compile(hipcc, src, obj_dir, verbose), SOURCES))
    tmp = LIB_PATH + ".tmp"
    link = subprocess.run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", tmp],
                          capture_output=True, text=True)
    if link.returncode != 0:
        raise RuntimeError(f"linking libcute_hip.so failed:\n{link.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


def kernel_resources(source: str, loops: bool = False) -> dict[str, dict[str, int]]:
    """Registers and scratch of every kernel of one source, as the compiler reports them
    (``-Rpass-analysis=kernel-resource-usage``): {mangled name: {"vgprs": n, "agprs": n, "scratch": bytes per lane}}.
    Scratch above zero means the kernel spills registers to memory.  With ``loops``, the device assembly of the same
    compilation is read as well and every kernel gets ``"loops"``: one dict per innermost loop that holds matrix
    instructions, counting them ("mfma") and what must not sit beside them - scratch accesses ("scratch") and copies
    between the two halves of the register file ("acc_moves") - plus LDS reads, direct-to-LDS copies and barriers."""
    import re
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "out.s" if loops else "out.o")
        mode = ["--cuda-device-only", "-S"] if loops else ["-c"]
        cmd = [find_hipcc(), *HIPCC_FLAGS, "-Rpass-analysis=kernel-resource-usage", *mode,
               os.path.join(CSRC_DIR, source), "-o", out]
        result = subprocess.run(cmd, capture_output=True, text=True)
        if result.returncode != 0:
            raise RuntimeError(f"hipcc failed on {source}:\n{result.stderr}")
        assembly = open(out).read().split("\n") if loops else []
    found: dict[str, dict[str, int]] = {}
    name = None
    for line in result.stderr.splitlines():
        if match := re.search(r"Function Name: (\S+)", line):
            name = match.group(1)
            found[name] = {}
        elif name and (match := re.search(r"remark:\s+VGPRs: (\d+)", line)):
            found[name]["vgprs"] = int(match.group(1))
        elif name and (match := re.search(r"remark:\s+AGPRs: (\d+)", line)):
            found[name]["agprs"] = int(match.group(1))
        elif name and (match := re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)):
            found[name]["scratch"] = int(match.group(1))
    if loops:
        starts = [(i, line.split(":")[0]) for i, line in enumerate(assembly) if re.match(r"^_Z\w+:", line)]
        for k, (first, kernel) in enumerate(starts):
            if kernel not in found:
                continue
            body = assembly[first:starts[k + 1][0] if k + 1 < len(starts) else len(assembly)]
            labels = {m.group(1): i for i, line in enumerate(body) if (m := re.match(r"^(\.LBB\d+_\d+):", line))}
            spans = []
            for i, line in enumerate(body):
                m = re.search(r"s_cbranch_\w+ (\.LBB\d+_\d+)", line)
                if m and labels.get(m.group(1), i) < i:
                    spans.append((labels[m.group(1)], i))
            innermost = [s for s in spans if not any(o != s and s[0] <= o[0] and o[1] <= s[1] for o in spans)]
            found[kernel]["loops"] = []
            for lo, hi in innermost:
                text = body[lo:hi]
                count = lambda word: sum(word in line for line in text)
                if count("v_mfma") > 0:
                    found[kernel]["loops"].append({
                        "mfma": count("v_mfma"), "scratch": count("scratch_"), "acc_moves": count("v_accvgpr"),
                        "lds_reads": count("ds_read"), "copies": count("global_load_lds"), "barriers": count("s_barrier"),
                    })
    return found


if __name__ == "__main__":
    print(build(verbose=True))
