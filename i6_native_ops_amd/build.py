"""Builds the native parts in-tree: libi6fbw.so (HIP kernels + C ABI, hipcc, gfx950) and the
PyTorch-ROCm bindings fbw_core and fast_viterbi_core (both link libi6fbw.so).  Takes the place of the reference's
setup.py FBW entry (setup.py:29-33) and its import-time JIT fallback (fbw/__init__.py:10-24):
nothing is compiled at import time, and nothing is hipified."""
import os
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
OUT = os.path.join(PKG, "fbw")
LIB = os.path.join(OUT, "libi6fbw.so")
EXT = os.path.join(OUT, "fbw_core" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# packed-fp32 code generation is switched off for all device code
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def kernel_resources(remarks):
    """{kernel name: {"vgprs": n, "scratch": bytes per lane, "occupancy": waves per SIMD}} from the compiler's
    kernel-resource-usage remarks"""
    import re
    out, cur = {}, None
    for line in remarks.splitlines():
        m = re.search(r"remark: Function Name: (\S+)", line)
        if m:
            cur = out.setdefault(m.group(1), {})
            continue
        for key, pat in (("vgprs", r"remark:\s+VGPRs: (\d+)"), ("scratch", r"ScratchSize \[bytes/lane\]: (\d+)"),
                         ("occupancy", r"Occupancy \[waves/SIMD\]: (\d+)")):
            m = re.search(pat, line)
            if m and cur is not None:
                cur[key] = int(m.group(1))
    return out


def sources_digest():
    """sha256 over the device sources and the compiler flags: kept inside kernel_resources.json, so that a record
    made from other sources than the ones present is recognised as such"""
    import hashlib
    h = hashlib.sha256(" ".join(HIP_FLAGS).encode())
    for name in sorted(os.listdir(CSRC)):
        if name.endswith((".hip", ".inc", ".h")):
            h.update(name.encode())
            h.update(open(os.path.join(CSRC, name), "rb").read())
    return h.hexdigest()


def build_lib(out_root=PKG):
    """libi6fbw.so into <out_root>/fbw (out_root: this package in the source tree, or its copy in a build tree),
    and beside it kernel_resources.json: registers, scratch and occupancy of every kernel as the compiler reports
    them (a kernel that outgrows its register budget spills without a word and runs at half its speed;
    tests/test_boundary_cpu.py reads this record)."""
    import json
    lib = os.path.join(out_root, "fbw", "libi6fbw.so")
    os.makedirs(os.path.dirname(lib), exist_ok=True)
    cmd = [HIPCC, *HIP_FLAGS, "-shared", "-Rpass-analysis=kernel-resource-usage", os.path.join(CSRC, "fbw_kernels.hip"), "-o", lib]
    print(" ".join(cmd), flush=True)
    done = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    remarks = done.stdout
    import re
    other = [l for l in remarks.splitlines()
             if "-Rpass-analysis=kernel-resource-usage" not in l and not re.match(r"^\s*(\d+ )?\|", l)]     # (and the source lines quoted with them)
    if other:
        print("\n".join(other), flush=True)
    if done.returncode != 0:
        raise subprocess.CalledProcessError(done.returncode, cmd)
    record = kernel_resources(remarks)
    record["_sources_sha256"] = sources_digest()
    with open(os.path.join(out_root, "fbw", "kernel_resources.json"), "w") as f:
        json.dump(record, f, indent=1, sort_keys=True)
    return lib


def build_ext(name="fbw_core", source="fbw_torch.cpp", out_dir=None, lib_dir=None):
    import torch
    from torch.utils import cpp_extension
    inc = cpp_extension.include_paths()
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=" + name, "-DTORCH_API_INCLUDE_EXTENSION_H",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-I" + sysconfig.get_paths()["include"], "-I/opt/rocm/include"]
    cmd += ["-I" + p for p in inc]
    out_dir = out_dir or OUT
    os.makedirs(out_dir, exist_ok=True)
    ext = os.path.join(out_dir, name + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))
    cmd += [os.path.join(CSRC, source), "-o", ext,
            "-L" + (lib_dir or OUT), "-li6fbw", "-L" + torch_lib, "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip",
            "-ltorch_python", "-L/opt/rocm/lib", "-lamdhip64",
            "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,$ORIGIN/../fbw", "-Wl,-rpath," + torch_lib, "-Wl,-rpath,/opt/rocm/lib", "-Wno-attributes"]
    _run(cmd)
    return ext


def build_all(out_root=PKG):
    """Everything native, into the package directory out_root (default: in the source tree)."""
    build_lib(out_root)
    lib_dir = os.path.join(out_root, "fbw")
    build_ext("fbw_core", "fbw_torch.cpp", lib_dir, lib_dir)
    build_ext("fast_viterbi_core", "viterbi_torch.cpp", os.path.join(out_root, "fast_viterbi"), lib_dir)


if __name__ == "__main__":
    build_all()
    sys.exit(0)
