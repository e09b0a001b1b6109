"""Builds every kernel source of the library for the host, against the workgroup emulation of tests/host/shim, into one
shared object with the library's own C entry points (`ck_*`, same signatures): the device code then runs on the CPU,
one coroutine per lane, and the tests call it through the package's ctypes binding on CPU tensors.

Test infrastructure only: nothing in the package loads it, and the package still refuses CPU tensors."""

import concurrent.futures
import contextlib
import ctypes
import glob
import os
import shutil
import subprocess


HOST_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(os.path.dirname(os.path.dirname(HOST_DIR)), "kernel-hyperdrive_amd", "csrc")
FLAGS = ["-std=c++17", "-O0", "-fPIC", "-x", "c++", "-I", os.path.join(HOST_DIR, "shim"), "-include",
         os.path.join(HOST_DIR, "shim", "ck_gemm_prims_emulated.h"), "-Wno-unknown-attributes", "-Wno-ignored-attributes",
         "-Wno-unused-value", "-Wno-psabi"]


def host_clang():
    """The kernel sources use clang's vector extensions and __bf16: the host compiler is the ROCm toolchain's clang."""
    for candidate in (shutil.which("amdclang++"), "/opt/rocm/llvm/bin/clang++", "/opt/rocm/bin/amdclang++"):
        if candidate and os.path.exists(candidate):
            return candidate
    return None


def build(directory: str, sources=None) -> str:
    """Compiles csrc/*.hip (or `sources`) and links libcute_hip_emulated.so in `directory`; returns its path."""
    compiler = host_clang()
    if compiler is None:
        raise RuntimeError("no clang of the ROCm toolchain to build the host emulation with")
    sources = sorted(sources or glob.glob(os.path.join(CSRC, "*.hip"))) + [os.path.join(HOST_DIR, "emulated_support.cpp")]
    objects = [os.path.join(directory, os.path.basename(s) + ".o") for s in sources]

    def compile_one(pair):
        source, obj = pair
        subprocess.run([compiler, *FLAGS, "-c", source, "-o", obj], check=True, capture_output=True, text=True)

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        list(pool.map(compile_one, zip(sources, objects)))
    library = os.path.join(directory, "libcute_hip_emulated.so")
    subprocess.run([compiler, "-shared", "-o", library, *objects], check=True, capture_output=True, text=True)
    return library


class _HostLaunch:
    """Stands in for the binding's launch context: no device to make current, no stream."""

    stream = None

    def __init__(self, *tensors):
        pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


def _with_aligned_workspace(function, pointer_at: int, bytes_at: int):
    """GPU allocations start on 256-byte boundaries and ck_embedding_backward checks that of its workspace; a CPU tensor
    starts on a 64-byte one.  The workspace is scratch (nothing in it before or after the call matters): the call gets
    an aligned buffer of the same size instead."""

    def call(*args):
        args = list(args)
        if args[pointer_at] and args[pointer_at] % 256:
            scratch = ctypes.create_string_buffer(args[bytes_at] + 256)
            args[pointer_at] = (ctypes.addressof(scratch) + 255) // 256 * 256
        return function(*args)

    return call


@contextlib.contextmanager
def bound_to(library: str):
    """While active, the package's ctypes binding (cute_kernels._C) calls the emulated library and takes CPU tensors."""
    from cute_kernels import _C

    lib = ctypes.CDLL(library)
    for name, (restype, argtypes) in _C._SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    from cute_kernels.cutotune import tuner

    lib.ck_embedding_backward = _with_aligned_workspace(lib.ck_embedding_backward, 4, 5)
    saved = (_C._lib, _C._Launch, _C.rmsnorm_backward_workspace_size, tuner._DISABLE_CUTOTUNE)
    _C._lib, _C._Launch = lib, _HostLaunch
    _C.rmsnorm_backward_workspace_size = lambda B, H, device: lib.ck_rmsnorm_backward_workspace_size(B, H)
    # nothing to time here: every tuned launcher takes its default configuration (the tests name other ones explicitly)
    tuner._DISABLE_CUTOTUNE = True
    try:
        yield lib
    finally:
        _C._lib, _C._Launch, _C.rmsnorm_backward_workspace_size, tuner._DISABLE_CUTOTUNE = saved
