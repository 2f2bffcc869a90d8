import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_addoption(parser):
    parser.addoption(
        "--on-emulation",
        action="store_true",
        help="run the tests marked gpu against the CPU emulation of the kernels (tests/emu) on a host without a GPU: "
        "the same test bodies and host code, the kernel sources compiled for the CPU; no substitute for the run on a GPU",
    )


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU (run on the GPU box with -m gpu)")


def _emulated_device():
    """The library of tests/emu in the place of libzorro_fca.so, and host tensors posing as device
    tensors: the host code under test checks ``is_cuda``, asks for the current stream and
    synchronises, none of which a host without a GPU can answer.  Only ever under --on-emulation,
    in a process of its own (tests/test_gpu_tests_on_emulation.py starts one)."""
    import ctypes

    import torch

    sys.path.insert(0, os.path.join(ROOT, "tests", "emu"))
    import build as emu_build

    import arctic_platform_amd.cache
    import arctic_platform_amd.forest
    import arctic_platform_amd.ops
    import arctic_platform_amd.reconstruct
    import arctic_platform_amd.split_attention
    from arctic_platform_amd import _lib

    if emu_build.compiler() is None:
        pytest.skip("no clang++ to build the emulation with")
    lib = _lib.declare_signatures(ctypes.CDLL(emu_build.build()))
    lib.emu_set_run_order(int(os.environ.get("FCA_EMU_RUN_ORDER", "0")))  # (see tests/test_emulated_kernels.py)
    lib.emu_set_host_threads(int(os.environ.get("FCA_EMU_THREADS", "1")))
    _lib.load_library = lambda: lib
    for module in ("cache", "forest", "ops", "reconstruct", "split_attention"):
        setattr(getattr(arctic_platform_amd, module), "_stream_ptr", lambda device: None)
    # a layout's device copy: "cuda" is the default of SplitLayout and what the tests pass
    layout_init = arctic_platform_amd.split_attention.SplitLayout.__init__

    def layout_on_the_host(self, groups, device="cuda", *args, **kwargs):
        layout_init(self, groups, "cpu", *args, **kwargs)
        self.dev = torch.from_numpy(self.host)

    arctic_platform_amd.split_attention.SplitLayout.__init__ = layout_on_the_host
    torch.Tensor.is_cuda = property(lambda self: True)
    torch.Tensor.cuda = lambda self, *args, **kwargs: self.clone()  # (a copy, as the transfer to a device is)
    torch.cuda.synchronize = lambda *args, **kwargs: None
    import types

    torch.cuda.get_device_properties = lambda device=None: types.SimpleNamespace(multi_processor_count=8, name="CPU emulation")  # (emu.h: 8 CUs)
    return torch.device("cpu")


_emulated = None


@pytest.fixture(scope="session", autouse=True)
def _emulation_if_asked_for(request):
    """(Some tests marked gpu take no ``gpu`` fixture and call ``.cuda()`` themselves.)"""
    global _emulated
    if request.config.getoption("--on-emulation"):
        import torch

        if torch.cuda.is_available():
            pytest.fail("--on-emulation is for hosts without a GPU; here the tests run on the GPU")
        _emulated = _emulated_device()
    yield


@pytest.fixture(scope="session")
def gpu(request):
    import torch

    if request.config.getoption("--on-emulation"):
        return _emulated
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this process")
    from arctic_platform_amd import _lib

    _lib.load_library()  # fails loudly if the HIP library was not built
    return torch.device("cuda:0")
