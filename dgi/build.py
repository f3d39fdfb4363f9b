"""Build the gfx950 extension in-tree: ``python -m dgi.build``
(``--sanitize``: the ASan+UBSan and TSan builds of the host ring code instead).

Each ``dgi/csrc/*.hip`` file is compiled by ``hipcc --offload-arch=gfx950``
into an object, ``bindings.cpp`` (torch op registration) is compiled against
the installed PyTorch-ROCm headers, and everything is linked into
``dgi/_C.so``.  No hipify step, no cpp_extension JIT cache: the ``.so`` sits
next to the sources so it travels with the repo snapshot to the GPU box.
"""
from __future__ import annotations

import concurrent.futures as cf
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
BUILD = os.path.join(HERE, "..", "build", "dgi_obj")
OUT = os.path.join(HERE, "_C.so")
ARCH = os.environ.get("DGI_OFFLOAD_ARCH", "gfx950")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _torch_paths():
    import torch

    root = os.path.dirname(torch.__file__)
    inc = [os.path.join(root, "include"), os.path.join(root, "include", "torch", "csrc", "api", "include")]
    lib = os.path.join(root, "lib")
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    return inc, lib, abi


def _newer(src_list, target):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in src_list)


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("command failed:\n" + " ".join(cmd) + "\n" + r.stdout + r.stderr)
    return r


# hipcc device-code flags: no packed-fp32 VALU forms (the compiler otherwise makes them from
# ordinary float code); the host pass warns that it does not know the feature, harmlessly
DEVICE_FLAGS = ["-munsafe-fp-atomics", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]

# extension libraries: name -> (source folder, output).  "core" is every kernel of the Llama-family
# runtime (dgi/_C.so); "mix" the mixer-block kernels of the per-layer-geometry models
# (dgi/_C_mix.so: norms, q/k norm + rotary, masked attention, activations), which builds in
# seconds so a model that needs only those does not wait for the big GEMM kernels.
GROUPS = {"core": (CSRC, OUT), "mix": (os.path.join(CSRC, "mix"), os.path.join(HERE, "_C_mix.so"))}


def build(verbose: bool = False, force: bool = False, group: str = "core") -> str:
    src_dir, out = GROUPS[group]
    obj_dir = BUILD if group == "core" else BUILD + "_" + group
    os.makedirs(obj_dir, exist_ok=True)
    inc, lib, abi = _torch_paths()
    hdrs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hdrs += [os.path.join(src_dir, f) for f in os.listdir(src_dir) if f.endswith(".h") and src_dir != CSRC]
    kernels = sorted(f for f in os.listdir(src_dir) if f.endswith(".hip"))
    sources = [os.path.join(src_dir, f) for f in os.listdir(src_dir) if f.endswith((".hip", ".cpp", ".cc"))]
    if not force and not _newer(sources + hdrs, out):
        return out      # the library is newer than every source (object files need not travel with it)
    common = ["-O3", "-fPIC", "-std=c++17", f"-D_GLIBCXX_USE_CXX11_ABI={abi}"]
    jobs = []
    objs = []
    for k in kernels:
        src = os.path.join(src_dir, k)
        obj = os.path.join(obj_dir, k + ".o")
        objs.append(obj)
        if force or _newer([src] + hdrs, obj):
            jobs.append([HIPCC, f"--offload-arch={ARCH}", *common, *DEVICE_FLAGS, "-c", src, "-o", obj])
    bsrc = os.path.join(src_dir, "bindings.cpp")
    bobj = os.path.join(obj_dir, "bindings.o")
    objs.append(bobj)
    py_inc = sysconfig.get_paths()["include"]
    if force or _newer([bsrc], bobj):
        jobs.append([HIPCC, *common, "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=_C",
                     *[f"-I{p}" for p in inc], f"-I{py_inc}", "-I/opt/rocm/include", "-x", "c++", "-c", bsrc, "-o", bobj])
    # native runtime pieces (C++ only)
    for f in sorted(os.listdir(src_dir)):
        if f.endswith(".cc"):
            src = os.path.join(src_dir, f)
            obj = os.path.join(obj_dir, f + ".o")
            objs.append(obj)
            if force or _newer([src] + hdrs, obj):
                jobs.append(["g++", *common, f"-I{py_inc}", *[f"-I{p}" for p in inc], "-c", src, "-o", obj])
    workers = int(os.environ.get("MAX_JOBS", "8"))
    with cf.ThreadPoolExecutor(max_workers=max(1, min(workers, 16))) as ex:
        for r in ex.map(_run, jobs):
            if verbose and r.stderr:
                print(r.stderr, file=sys.stderr)
    if force or jobs or not os.path.exists(out):
        tmp = out + f".tmp{os.getpid()}"
        _run([HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", tmp, f"-L{lib}",
              "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip", f"-Wl,-rpath,{lib}"])
        os.replace(tmp, out)
    return out


SHM_SRC = os.path.join(CSRC, "host", "shm_ring.cc")
SHM_OUT = os.path.join(HERE, "_shm" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_shm(force: bool = False) -> str:
    """``dgi/_shm*.so``: the shared-memory control-plane rings (plain C++ /
    pybind11, no ROCm dependency, so the CPU test-suite uses the same code)."""
    if not force and not _newer([SHM_SRC, os.path.join(CSRC, "host", "shm_ring.h")], SHM_OUT):
        return SHM_OUT
    import pybind11
    py_inc = sysconfig.get_paths()["include"]
    _run(["g++", "-O2", "-fPIC", "-shared", "-std=c++17", "-Wall", f"-I{pybind11.get_include()}", f"-I{py_inc}",
          SHM_SRC, "-o", SHM_OUT, "-lrt"])
    return SHM_OUT


STRESS_SRC = os.path.join(CSRC, "host", "shm_ring_stress.cc")
SANITIZERS = {
    # ASan + UBSan: bounds of every ring copy against the mapping, misaligned cursor access
    "asan": ["-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-fno-omit-frame-pointer"],
    # TSan: the producer / consumer cursor protocol (release / acquire) on one mapping
    "tsan": ["-fsanitize=thread"],
}


def build_sanitized(kind: str, force: bool = False, defines: tuple = (), tag: str = "") -> str:
    """CPU sanitizer build of the native host code: the shared-memory ring
    core (``csrc/host/shm_ring.h``, the one concurrent native component) linked into the
    stress driver ``shm_ring_stress.cc`` with ``SANITIZERS[kind]``; returns the binary's path
    (``build/sanitize/shm_ring_stress_<kind>``).  Host code only: no GPU code is sanitized."""
    flags = SANITIZERS[kind]
    out_dir = os.path.join(HERE, "..", "build", "sanitize")
    os.makedirs(out_dir, exist_ok=True)
    out = os.path.join(out_dir, f"shm_ring_stress_{kind}{tag}")
    hdr = os.path.join(CSRC, "host", "shm_ring.h")
    if force or _newer([STRESS_SRC, hdr], out):
        _run(["g++", "-O1", "-g", "-std=c++17", "-Wall", "-Wextra", *flags, *[f"-D{d}" for d in defines],
              STRESS_SRC, "-o", out, "-lrt", "-pthread"])
    return out


if __name__ == "__main__":
    if "--sanitize" in sys.argv:
        for k in SANITIZERS:
            print(build_sanitized(k, force="--force" in sys.argv))
        sys.exit(0)
    print(build_shm(force="--force" in sys.argv))
    groups = [g for g in GROUPS if g in sys.argv] or list(GROUPS)
    for g in groups:
        print(build(verbose=True, force="--force" in sys.argv, group=g))
