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
    between the two halves of the register file ("acc_moves") - plus LDS reads, direct-to-LDS copies and barriers; and
    ``"unsettled"``: the instructions that touch an accumulation register fewer than 19 wait states behind a matrix
    instruction issued through ``asm`` on some path (see ``_unsettled_accumulator_accesses``)."""
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
            found[kernel]["unsettled"] = _unsettled_accumulator_accesses(body)
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


def _unsettled_accumulator_accesses(body: list[str], settled: int = 19) -> list[str]:
    """A matrix instruction writes its result several passes after it issues, and the hardware does not hold back a
    vector-ALU or memory instruction that reads (or overwrites) the register earlier: the compiler counts wait states
    and pads with ``s_nop`` - for the matrix instructions it knows.  One written in ``asm`` is text to it.  This walks
    the control-flow graph of one kernel's assembly and reports every instruction other than a matrix instruction that
    names an accumulation register and can be reached from an ``asm`` matrix instruction in fewer than ``settled`` wait
    states (one per instruction, ``s_nop n`` counting n + 1; 18 is the longest requirement, of a 16-pass instruction)."""
    import re

    blocks: list[dict] = [{"label": None, "code": []}]
    in_asm = False
    for line in body[1:]:
        text = line.split(";")[0].rstrip() if not line.lstrip().startswith(";;#") else line.strip()
        if text.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if text.startswith(";;#ASMEND"):
            in_asm = False
            continue
        if match := re.match(r"^(\.LBB\d+_\d+):", line):
            blocks.append({"label": match.group(1), "code": []})
            continue
        if not line.startswith("\t") or not text.strip() or text.strip().startswith("."):
            continue
        blocks[-1]["code"].append((text.strip(), in_asm))
        if re.match(r"^(s_branch|s_cbranch_\w+|s_endpgm|s_setpc_b64)\b", text.strip()):
            blocks.append({"label": None, "code": []})
    index = {b["label"]: i for i, b in enumerate(blocks) if b["label"]}
    successors: list[list[int]] = []
    for i, b in enumerate(blocks):
        last = b["code"][-1][0] if b["code"] else ""
        nxt = [i + 1] if i + 1 < len(blocks) else []
        if match := re.match(r"^s_branch (\S+)", last):
            successors.append([index[match.group(1)]] if match.group(1) in index else [])
        elif match := re.match(r"^s_cbranch_\w+ (\S+)", last):
            successors.append(nxt + ([index[match.group(1)]] if match.group(1) in index else []))
        elif re.match(r"^(s_endpgm|s_setpc_b64)", last):
            successors.append([])
        else:
            successors.append(nxt)

    def registers(text: str) -> set[int]:
        named: set[int] = set()
        for lo, hi in re.findall(r"\ba\[(\d+):(\d+)\]", text):
            named.update(range(int(lo), int(hi) + 1))
        named.update(int(n) for n in re.findall(r"\ba(\d+)\b", text))
        return named

    # state: accumulation register -> wait states since an asm matrix instruction wrote it (absent: settled)
    def walk(i: int, state: dict[int, int], report: list[str] | None) -> dict[int, int]:
        state = dict(state)
        for text, from_asm in blocks[i]["code"]:
            if text.startswith("v_mfma"):
                if from_asm:
                    for reg in registers(text.split(",")[0]):
                        state[reg] = 0
                    continue
            elif state and report is not None:
                early = {reg: state[reg] for reg in registers(text) if reg in state}
                if early:
                    report.append(f"{text}  ({min(early.values())} wait states behind the matrix instruction that wrote it)")
            step = int(text.split()[1]) + 1 if text.startswith("s_nop") else 1
            state = {reg: d + step for reg, d in state.items() if d + step < settled}
        return state

    entry: list[dict[int, int]] = [{} for _ in blocks]
    changed = True
    while changed:
        changed = False
        for i in range(len(blocks)):
            out = walk(i, entry[i], None)
            for j in successors[i]:
                for reg, d in out.items():
                    if d < entry[j].get(reg, settled):
                        entry[j][reg] = d
                        changed = True
    found: list[str] = []
    for i in range(len(blocks)):
        walk(i, entry[i], found)
    return found


if __name__ == "__main__":
    print(build(verbose=True))
