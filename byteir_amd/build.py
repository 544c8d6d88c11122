"""Builds the in-tree shared libraries with hipcc for gfx950 (no GPU needed to compile).

    python -m byteir_amd.build            # build everything
    python -m byteir_amd.build kernels    # one target

Targets:
  kernels -> lib/libbrt_rocm_kernels.so   reductions, softmax, device plumbing (C ABI)
  flash   -> lib/libflash_attn.so         flash-attention custom library (C ABI)
  brt     -> lib/libbrt.so                BRT-shaped C++ host runtime (g++, no HIP headers)
  index_check -> lib/libfa_index_check.so host-only bounds check of the flash-attention index arithmetic
"""
import os
import subprocess
import sys
import time

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "lib")
INC = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -packed-fp32-ops is switched off on purpose: the compiler must not form v_pk_*_f32.
HIP_FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-shared",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             "-Wno-unused-command-line-argument", f"-I{INC}"]
CXX_FLAGS = ["-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", f"-I{INC}"]


def _glob(sub, exts):
    d = os.path.join(CSRC, sub)
    return sorted(os.path.join(d, f) for f in os.listdir(d) if f.endswith(exts))


def _run(cmd, verbose):
    t = time.time()
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("build failed: " + " ".join(cmd) + "\n" + out)
    if verbose:
        print(f"[build] {os.path.basename(cmd[cmd.index('-o') + 1])} in {time.time() - t:.1f}s")
        if out.strip():
            print(out)


def build_kernels(verbose=False):
    os.makedirs(LIB, exist_ok=True)
    _run([HIPCC] + HIP_FLAGS + ["-o", os.path.join(LIB, "libbrt_rocm_kernels.so")] + _glob("kernels", (".hip",)), verbose)


def build_flash(verbose=False):
    os.makedirs(LIB, exist_ok=True)
    _run([HIPCC] + HIP_FLAGS + [f"-I{os.path.join(CSRC, 'flash_attn')}", "-o", os.path.join(LIB, "libflash_attn.so")]
         + _glob("flash_attn", (".hip",)), verbose)


def build_brt(verbose=False):
    os.makedirs(LIB, exist_ok=True)
    srcs = _glob("brt", (".cc",))
    if not srcs:
        return
    _run(["g++"] + CXX_FLAGS + [f"-I{os.path.join(CSRC, 'brt')}", "-o", os.path.join(LIB, "libbrt.so")] + srcs
         + [f"-L{LIB}", "-lbrt_rocm_kernels", "-ldl", "-Wl,-rpath,$ORIGIN"], verbose)


def build_index_check(verbose=False):
    """Host-only bounds check of the flash-attention kernels' index arithmetic (g++, no GPU)."""
    os.makedirs(LIB, exist_ok=True)
    _run(["g++"] + CXX_FLAGS + ["-o", os.path.join(LIB, "libfa_index_check.so"),
                                os.path.join(CSRC, "flash_attn", "index_check.cc")], verbose)


def build_test_kernels(verbose=False):
    """The external op-kernel library of the tests (tests/external_kernels/custom_add.hip, in the
    style of the reference's runtime/test/external_kernels): built here, ahead of time, so that
    the GPU tests only load it."""
    src = os.path.join(ROOT, "tests", "external_kernels", "custom_add.hip")
    if not os.path.exists(src):
        return
    _run([HIPCC] + HIP_FLAGS + [f"-I{os.path.join(CSRC, 'brt')}", "-o",
                                os.path.join(ROOT, "tests", "external_kernels", "libcustom_add.so"), src,
                                f"-L{LIB}", "-lbrt", "-lbrt_rocm_kernels", f"-Wl,-rpath,{LIB}"], verbose)


def build_emu(verbose=False):
    """The three libraries once more, for the host: the .hip sources compiled unchanged by a host
    clang against tests/emu/wave_emu.h (which stands in for the HIP runtime header and runs every
    lane as a fiber), a host stand-in for the device layer, and the runtime linked against them
    -- tests/emu/lib/{libbrt_rocm_kernels,libflash_attn,libbrt}.so, the same C ABIs on host
    memory, for the tests that need no GPU.  Needs a host clang (vector extensions, _Float16,
    __bf16); skipped when there is none.  Nothing in the package loads these."""
    clang = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "llvm", "bin", "clang++")
    emu = os.path.join(ROOT, "tests", "emu")
    if not os.path.exists(clang) or not os.path.isdir(emu):
        return
    import concurrent.futures
    obj, out = os.path.join(emu, "obj"), os.path.join(emu, "lib")
    os.makedirs(obj, exist_ok=True)
    os.makedirs(out, exist_ok=True)
    flags = ["-std=c++17", "-O2", "-fPIC", "-DFA_EMULATE", f"-I{os.path.join(emu, 'include')}", f"-I{emu}",
             f"-I{os.path.join(CSRC, 'flash_attn')}", f"-I{os.path.join(CSRC, 'kernels')}", f"-I{os.path.join(ROOT, 'include')}",
             "-Wno-unknown-attributes", "-ffp-contract=off"]
    attn = [(src, os.path.join(obj, os.path.basename(src) + ".o"), ["-x", "c++"]) for src in _glob("flash_attn", (".hip",))]
    # the reductions, the softmax and the input generator; device.hip is the HIP runtime plumbing:
    # tests/emu/device_emu.cc takes its place
    kern = [(os.path.join(CSRC, "kernels", n + ".hip"), os.path.join(obj, n + ".hip.o"), ["-x", "c++"]) for n in ("reduce", "softmax", "fill")]
    kern.append((os.path.join(emu, "device_emu.cc"), os.path.join(obj, "device_emu.o"), []))
    rt = [(os.path.join(emu, "wave_emu.cc"), os.path.join(obj, "wave_emu.o"), [])]
    with concurrent.futures.ThreadPoolExecutor(max_workers=8) as pool:
        list(pool.map(lambda j: _run([clang] + j[2] + flags + ["-c", j[0], "-o", j[1]], False), attn + kern + rt))
    # -Bsymbolic: a library's own calls stay inside it whatever else the process has loaded
    _run([clang, "-shared", "-fPIC", "-Wl,-Bsymbolic", "-o", os.path.join(out, "libflash_attn.so")] + [j[1] for j in attn + rt], verbose)
    _run([clang, "-shared", "-fPIC", "-Wl,-Bsymbolic", "-Wl,--no-undefined", "-o", os.path.join(out, "libbrt_rocm_kernels.so")]
         + [j[1] for j in kern + rt], verbose)
    srcs = _glob("brt", (".cc",))
    if srcs:
        _run(["g++"] + CXX_FLAGS + [f"-I{os.path.join(CSRC, 'brt')}", "-o", os.path.join(out, "libbrt.so")] + srcs
             + [f"-L{out}", "-lbrt_rocm_kernels", "-ldl", "-Wl,-rpath,$ORIGIN"], verbose)


TARGETS = {"kernels": build_kernels, "flash": build_flash, "brt": build_brt, "index_check": build_index_check,
           "test_kernels": build_test_kernels, "emu": build_emu}


def build_all(verbose=False, targets=None):
    for name in targets or ("kernels", "flash", "brt", "index_check", "test_kernels", "emu"):
        TARGETS[name](verbose)


if __name__ == "__main__":
    build_all(verbose=True, targets=sys.argv[1:] or None)
