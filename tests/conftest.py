import os
import sys

import pytest


ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for path in (ROOT, os.path.join(ROOT, "kernel-hyperdrive_amd")):
    if path not in sys.path:
        sys.path.insert(0, path)

os.environ.setdefault("DEBUG_CUTEINDUCTOR", "0")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_addoption(parser):
    parser.addoption("--emulated-device", action="store_true",
                     help="give the tests marked gpu the CPU emulation of the kernels (tests/host) as their device: "
                          "no GPU needed, slow - problems beyond a few hundred rows take minutes")


@pytest.fixture(scope="session")
def gpu(request, tmp_path_factory):
    import torch

    if request.config.getoption("--emulated-device"):
        # every kernel source built for the host under the workgroup emulation, behind the package's own binding
        from host import emulated_library

        if emulated_library.host_clang() is None:
            pytest.skip("no clang of the ROCm toolchain to build the host emulation with")
        binding = emulated_library.bound_to(emulated_library.build(str(tmp_path_factory.mktemp("emulated_library"))),
                                            guarded=True)
        binding.__enter__()
        request.addfinalizer(lambda: binding.__exit__(None, None, None))
        return torch.device("cpu")
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda", 0)
