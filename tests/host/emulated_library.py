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

import torch


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
    flags, link = FLAGS, []
    if os.environ.get("EMULATED_LIBRARY_SANITIZE"):
        # The host's AddressSanitizer over the device code: LDS buffers are globals and per-lane arrays stack objects
        # here, so an index that leaves one is reported.  The runtime is a shared library that comes in with this one;
        # the process needs ASAN_OPTIONS=verify_asan_link_order=0:detect_leaks=0 and the directory of
        # libclang_rt.asan-x86_64.so (under the toolchain's lib/clang) on LD_LIBRARY_PATH.  Three minutes to build.
        sanitize = ["-fsanitize=address", "-shared-libsan", "-fno-omit-frame-pointer"]
        flags = [f for f in FLAGS if f != "-O0"] + ["-O1", "-g", *sanitize]
        link = sanitize
    objects = [os.path.join(directory, os.path.basename(s) + ".o") for s in sources]

    def compile_one(pair):
        source, obj = pair
        subprocess.run([compiler, *flags, "-c", source, "-o", obj], check=True, capture_output=True, text=True)

    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        list(pool.map(compile_one, zip(sources, objects)))
    library = os.path.join(directory, "libcute_hip_emulated.so")
    subprocess.run([compiler, "-shared", *link, "-o", library, *objects], check=True, capture_output=True, text=True)
    return library


_libc = ctypes.CDLL(None, use_errno=True)
_libc.mmap.restype = ctypes.c_void_p
_libc.mmap.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_long]
_libc.mprotect.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
_libc.munmap.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
_PAGE = 4096


class _GuardedCall:
    """One call into the library with every tensor moved, for its length, to memory that ends (within 15 bytes: the
    pointer keeps its alignment modulo 16, which the entry points branch on) at a page nobody may touch - or, with
    `before`, that begins right behind one: a kernel that
    reads or writes past the end of an operand - what faults a GPU, or silently corrupts a neighbour - ends the process
    with a segmentation fault here, and faulthandler names the test.  The contents travel back when the call returns."""

    def __init__(self, before: bool = False):
        self.before = before  # the inaccessible page lies before the operand instead of behind it
        self.regions = []  # (first byte, end) of the tensor's storage range, address of its guarded copy, mapping, size

    def pointer(self, t):
        if t is None:
            return None
        if t.numel() == 0:
            return t.data_ptr()
        nbytes = (sum((size - 1) * stride for size, stride in zip(t.shape, t.stride())) + 1) * t.element_size()
        lo, hi = t.data_ptr(), t.data_ptr() + nbytes
        for first, end, copy, _, _ in self.regions:
            if first <= lo and hi <= end:
                return copy + (lo - first)
            if lo < end and first < hi:
                raise RuntimeError("two operands of one call overlap in part: the guarded copies cannot stand for both")
        pages = (nbytes + 16 + _PAGE - 1) // _PAGE
        size = (pages + 1) * _PAGE
        mapping = _libc.mmap(None, size, 3, 0x22, -1, 0)  # PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS
        if mapping in (None, ctypes.c_void_p(-1).value):
            raise MemoryError("mmap")
        fence = mapping if self.before else mapping + pages * _PAGE
        if _libc.mprotect(fence, _PAGE, 0) != 0:
            raise OSError(ctypes.get_errno(), "mprotect")
        if self.before:
            copy = mapping + _PAGE + lo % 16
        else:
            copy = fence - nbytes
            copy -= (copy - lo) % 16
        if t.dtype == torch.uint8:
            # a workspace: its contents are undefined by contract, so a kernel that reads a byte of it before writing
            # it reads ones here (NaNs as floats, -1 as integers) and the results show it
            ctypes.memset(copy, 0xFF, nbytes)
        else:
            ctypes.memmove(copy, lo, nbytes)
        self.regions.append((lo, hi, copy, mapping, size))
        return copy

    def finish(self):
        for first, end, copy, mapping, size in self.regions:
            ctypes.memmove(first, copy, end - first)
            _libc.munmap(mapping, size)
        self.regions = []


_current_call = None


class _HostLaunch:
    """Stands in for the binding's launch context: no device to make current, no stream."""

    stream = None
    guarded = False  # False, True / "behind", or "before": where the inaccessible page lies

    def __init__(self, *tensors):
        pass

    def __enter__(self):
        global _current_call
        if self.guarded:
            _current_call = _GuardedCall(before=self.guarded == "before")
        return self

    def __exit__(self, *exc):
        global _current_call
        if _current_call is not None:
            _current_call.finish()
            _current_call = None
        return False


def _pointer(t):
    if _current_call is not None:
        return _current_call.pointer(t)
    return None if t is None else t.data_ptr()


def _with_aligned_workspace(function, pointer_at: int, bytes_at: int):
    """GPU allocations start on 256-byte boundaries and ck_embedding_backward checks that of its workspace; a CPU tensor
    starts on a 64-byte one.  The workspace is scratch (nothing in it before or after the call matters): the call gets
    an aligned buffer of the same size instead."""

    def call(*args):
        args = list(args)
        if args[pointer_at] and args[pointer_at] % 256:
            scratch = ctypes.create_string_buffer(args[bytes_at] + 256)
            ctypes.memset(scratch, 0xFF, args[bytes_at] + 256)  # (undefined contents: not zeros, which could pass for cleared)
            args[pointer_at] = (ctypes.addressof(scratch) + 255) // 256 * 256
        return function(*args)

    return call


@contextlib.contextmanager
def bound_to(library: str, guarded=False):
    """While active, the package's ctypes binding (cute_kernels._C) calls the emulated library and takes CPU tensors.
    `guarded` (True or "before"): every operand of every call sits in front of an inaccessible page, or right behind
    one (see _GuardedCall)."""
    from cute_kernels import _C

    lib = ctypes.CDLL(library)
    for name, (restype, argtypes) in _C._SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    from cute_kernels.cutotune import tuner

    lib.ck_embedding_backward = _with_aligned_workspace(lib.ck_embedding_backward, 4, 5)
    saved = (_C._lib, _C._Launch, _C.rmsnorm_backward_workspace_size, tuner._DISABLE_CUTOTUNE, _C._ptr, _HostLaunch.guarded)
    _C._lib, _C._Launch, _C._ptr, _HostLaunch.guarded = lib, _HostLaunch, _pointer, guarded
    _C.rmsnorm_backward_workspace_size = lambda B, H, device: lib.ck_rmsnorm_backward_workspace_size(B, H)
    # nothing to time here: every tuned launcher takes its default configuration (the tests name other ones explicitly)
    tuner._DISABLE_CUTOTUNE = True
    try:
        yield lib
    finally:
        (_C._lib, _C._Launch, _C.rmsnorm_backward_workspace_size, tuner._DISABLE_CUTOTUNE, _C._ptr,
         _HostLaunch.guarded) = saved
