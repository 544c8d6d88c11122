"""ByRE modules through the whole stack on a machine without a GPU: the runtime (session, plan,
frame, op kernels), linked against the host builds of the kernel libraries (tests/emu/lib: the
HIP kernels executed lane by lane, "device" memory = host memory behind protected pages).  The
reference's flash-attention test modules and golden vectors, its reduction shape list, the
Reduce* lines of its ResNet-18 modules and a host -> device -> host module all run as they do
on the GPU (tests/test_gpu_brt_session.py), each scenario in a process of its own
(tests/emu_session_child.py)."""
import os
import subprocess
import sys

import pytest

import emu_util as E

pytestmark = pytest.mark.skipif(not (os.path.exists(E.LIB) or os.path.exists("/opt/rocm/llvm/bin/clang++")),
                                reason="no host clang to build the emulated libraries with")


@pytest.mark.parametrize("scenario", ["reductions", "resnet_reduce_ops", "flash_attn_golden", "softmax_and_copies"])
def test_modules_run_through_the_session_on_the_host(scenario):
    E.lib()  # builds tests/emu/lib on demand
    child = os.path.join(os.path.dirname(os.path.abspath(__file__)), "emu_session_child.py")
    r = subprocess.run([sys.executable, child, scenario], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0 and f"ok {scenario}" in r.stdout, r.stdout[-2000:] + r.stderr[-4000:]


@pytest.mark.parametrize("header,lib", [("brt_rocm_kernels.h", "libbrt_rocm_kernels.so"), ("brt_rocm_bench.h", "libbrt_rocm_kernels.so"),
                                        ("flash_api.h", "libflash_attn.so"), ("brt_c_api.h", "libbrt.so")])
def test_the_host_builds_export_the_same_c_abi(header, lib):
    """Whatever include/*.h declares, the host build of the library exports too (a stand-in that
    cannot work on a host, e.g. launching a __global__ function of an external library, returns
    an error code)."""
    import ctypes
    from test_brt_host import exported_functions
    E.lib()
    if lib == "libbrt.so":  # its dependency is found through its rpath
        ctypes.CDLL(os.path.join(E.EMU_LIB_DIR, "libbrt_rocm_kernels.so"), mode=ctypes.RTLD_LOCAL)
    L = ctypes.CDLL(os.path.join(E.EMU_LIB_DIR, lib), mode=ctypes.RTLD_LOCAL)
    missing = [n for n in exported_functions(header) if not hasattr(L, n)]
    assert not missing, missing
