"""Builds the gfx950 shared libraries in-tree with hipcc / g++.

    python -m xfastertransformer_amd.build          # everything
The built .so files sit next to this package so that they travel with a source snapshot
to a GPU machine; nothing is installed into site-packages.
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
ROOT = os.path.dirname(HERE)
LIB_HIP = os.path.join(HERE, "libxft_hip.so")
LIB_LAYERS = os.path.join(HERE, "libxft_layers.so")
LIB_TORCH = os.path.join(HERE, "libxft_pt.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# gfx950 only; packed-FP32 VALU ops stay off (the compiler must not form v_pk_*_f32)
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-fno-gpu-rdc"]


def _run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def _stale(target, sources):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in sources)


def build_hip(force=True):
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    deps = srcs + glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(ROOT, "include", "*.h"))
    objdir = os.path.join(CSRC, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = []
    todo = []
    for s in srcs:
        o = os.path.join(objdir, os.path.basename(s) + ".o")
        objs.append(o)
        if force or _stale(o, [s] + [d for d in deps if d.endswith(".h")]):
            todo.append((s, [HIPCC] + HIP_FLAGS + ["-c", s, "-o", o]))
    # at most `jobs` compilers at a time (the template-heavy units take a minute or two each)
    jobs = max(1, min(8, os.cpu_count() or 1))
    failed = False
    running = []
    built = bool(todo)

    def reap(pr_s):
        nonlocal failed
        s, pr = pr_s
        out, _ = pr.communicate()
        out = "\n".join(l for l in out.splitlines() if "not a recognized feature" not in l)
        if out.strip():
            print(out)
        if pr.returncode != 0:
            failed = True
            print("FAILED:", s)

    while todo or running:
        while todo and len(running) < jobs:
            s, cmd = todo.pop(0)
            print("+", " ".join(cmd), flush=True)
            running.append((s, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        reap(running.pop(0))
    if failed:
        raise RuntimeError("hipcc failed")
    if force or built or not os.path.exists(LIB_HIP):
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_HIP] + objs)
    return LIB_HIP


def build_host(force=True):
    """The C++ host layer (xft::invoke* entry points, xft::AutoModel) over the C-ABI; plain g++, no HIP headers."""
    srcs = sorted(glob.glob(os.path.join(CSRC, "host", "*.cpp")))
    deps = srcs + glob.glob(os.path.join(CSRC, "host", "*.h")) + glob.glob(os.path.join(ROOT, "include", "*.h")) + [LIB_HIP]
    if force or _stale(LIB_LAYERS, deps):
        _run([os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall"] + srcs + ["-o", LIB_LAYERS,
              "-L" + HERE, "-lxft_hip", "-Wl,-rpath,$ORIGIN"])
    return LIB_LAYERS


def build_torch(force=True):
    """torch.classes.xfastertransformer.AutoModel over libxft_layers.so: g++ against the Torch headers of this
    interpreter's torch (no HIP code, no torch device memory: token ids and logits are host tensors)."""
    src = os.path.join(CSRC, "torch", "xft_torch.cpp")
    deps = [src, os.path.join(ROOT, "include", "models.h"), LIB_LAYERS]
    if not (force or _stale(LIB_TORCH, deps)):
        return LIB_TORCH
    import torch
    from torch.utils import cpp_extension
    inc = []
    for d in cpp_extension.include_paths():
        inc += ["-isystem", d]
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    abi = "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)
    _run([os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-variable", abi, src, "-o", LIB_TORCH]
         + inc + ["-L" + HERE, "-lxft_layers", "-lxft_hip", "-L" + tlib, "-ltorch", "-ltorch_cpu", "-lc10", "-Wl,-rpath,$ORIGIN",
                  "-Wl,-rpath," + tlib])
    return LIB_TORCH


def build_test_drivers(force=True):
    """C++ programs of the test suite that call the host API the way a program written against the reference's
    headers would (built here, not inside a GPU test)."""
    out = os.path.join(CSRC, "build", "set_input_driver")
    src = os.path.join(ROOT, "tests", "set_input_driver.cpp")
    if force or _stale(out, [src, LIB_LAYERS, os.path.join(ROOT, "include", "models.h")]):
        _run([os.environ.get("CXX", "g++"), "-O1", "-std=c++17", "-Wall", "-I" + os.path.join(ROOT, "include"), src, "-o", out, "-L" + HERE,
              "-lxft_layers", "-lxft_hip", "-Wl,-rpath," + HERE])
    return out


def build_all(force=True):
    build_hip(force)
    build_host(force)
    build_test_drivers(force)
    return build_torch(force)


if __name__ == "__main__":
    build_all(force="--incremental" not in sys.argv)
    print("built", LIB_HIP)
