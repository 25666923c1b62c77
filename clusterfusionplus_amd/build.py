"""In-tree build of the two native libraries (no JIT cache, no install step):

  libcfpp.so          HIP kernels + the C ABI of include/cfpp.h, compiled by hipcc for gfx950
  _clusterfusion.so   the PyTorch binding (host C++ only), compiled by g++ against libtorch

Both land next to this file so that they travel with the source tree.
`python -m clusterfusionplus_amd.build` rebuilds both.
"""
from __future__ import annotations

import os
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
INCLUDE = os.path.join(ROOT, "include")
LIB = os.path.join(PKG, "libcfpp.so")
EXT = os.path.join(PKG, "_clusterfusion.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed-fp32 arithmetic stays off in device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    # no contraction of a*b + c by the compiler: every fused multiply-add of the kernels is written out, so that a device
    # function rounds the same way in every kernel it is inlined into (split == fused, bit for bit)
    "-ffp-contract=off",
    # one name for the product build and for profiling builds kept elsewhere: a process that has loaded either one
    # resolves the binding's dependency on "libcfpp.so" to it
    "-Wl,-soname,libcfpp.so",
]


def _run(cmd):
    print("+ " + " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if out.strip():
        print(out, flush=True)
    if res.returncode != 0:
        raise RuntimeError(f"build command failed ({res.returncode}): {' '.join(cmd)}")


def build_lib(trace: bool = False, out: str = LIB):
    """libcfpp.so.  `trace`: a profiling build (-DCFPP_TRACE) whose fused kernel stores phase timestamps for
    `python clusterfusionplus_amd/phase_trace.py --trace-lib PATH`; it is slower by the stores, is written to a path
    of its own and never takes the place of the product library."""
    if trace and os.path.abspath(out) == os.path.abspath(LIB):
        raise ValueError("a profiling build must not overwrite the product library; give it a path of its own")
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    extra = ["-DCFPP_TRACE"] if trace else []
    _run([hipcc, *HIPCC_FLAGS, *extra, f"-I{INCLUDE}", f"-I{CSRC}", os.path.join(CSRC, "cfpp_kernels.hip"), "-o", out])
    return out


def resource_report(out=None):
    """Compiles the HIP library with the compiler's kernel-resource-usage remarks and returns one line per kernel:
    VGPRs, AGPRs, scratch bytes per lane (register spills), static LDS bytes per workgroup, waves per SIMD."""
    import re
    import tempfile
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    with tempfile.TemporaryDirectory() as tmp:
        cmd = [hipcc, *HIPCC_FLAGS, "-Rpass-analysis=kernel-resource-usage", f"-I{INCLUDE}", f"-I{CSRC}",
               os.path.join(CSRC, "cfpp_kernels.hip"), "-o", os.path.join(tmp, "libcfpp.so")]
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("resource report: compilation failed\n" + res.stdout[-2000:])
    rows = []
    for block in re.split(r"remark: [^\n]*Function Name: ", res.stdout)[1:]:
        name = block.split()[0]
        nice = subprocess.run(["c++filt", name], stdout=subprocess.PIPE, text=True).stdout.strip() or name
        if nice.startswith("_Z"):
            # c++filt does not know the _Float16 mangling (DF16_): take the kernel's name and its integer / bool template
            # arguments out of the mangled name by hand
            m = re.match(r"_ZN12_GLOBAL__N_1(\d+)", name)
            if m:
                n = int(m.group(1))
                base = name[m.end():m.end() + n]
                targs = re.match(r"I((?:L[ib]\d+E)+)E", name[m.end() + n:])
                if targs:
                    vals = [v if k == "i" else ("true" if v == "1" else "false") for k, v in re.findall(r"L([ib])(\d+)E", targs.group(1))]
                    base += "<" + ", ".join(vals) + ">"
                nice = base
        nice = nice.replace("(anonymous namespace)::", "").replace("void ", "")
        nice = re.sub(r"\(.*\)$", "", nice)

        def g(key):
            m = re.search(key + r": (\S+)", block)
            return m.group(1) if m else "?"
        rows.append((nice, g("VGPRs"), g("AGPRs"), g(r"ScratchSize \[bytes/lane\]"), g(r"LDS Size \[bytes/block\]"),
                     g(r"Occupancy \[waves/SIMD\]")))
    lines = [f"{'kernel':44s} {'VGPRs':>6s} {'AGPRs':>6s} {'scratch B/lane':>15s} {'LDS B/workgroup':>16s} {'waves/SIMD':>11s}"]
    lines += [f"{n[:44]:44s} {v:>6s} {a:>6s} {sc:>15s} {l:>16s} {o:>11s}" for n, v, a, sc, l, o in rows]
    text = "\n".join(lines)
    if out:
        with open(out, "w") as f:
            f.write(text + "\n")
    return text


def build_ext():
    import torch
    from torch.utils import cpp_extension as ce
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    incs = [f"-I{p}" for p in ce.include_paths("cuda")] + [f"-I{sysconfig.get_paths()['include']}", f"-I{INCLUDE}"]
    abi = int(torch.compiled_with_cxx11_abi())
    cmd = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wno-attributes",
        "-DUSE_ROCM", "-D__HIP_PLATFORM_AMD__=1", "-DTORCH_EXTENSION_NAME=_clusterfusion",
        "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={abi}",
        *incs, os.path.join(CSRC, "cfpp_torch.cpp"), "-o", EXT,
        f"-L{PKG}", "-lcfpp", f"-L{tlib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
        "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}",
    ]
    _run(cmd)
    return EXT


def build_stream_probe(out=os.path.join(PKG, "stream_probe_bin")):
    """The bare read probes (csrc/stream_probe.hip) as an executable next to this file; a measurement tool."""
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    _run([hipcc, "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-Wno-unused-command-line-argument", os.path.join(CSRC, "stream_probe.hip"), "-o", out])
    return out


def build_all():
    build_lib()
    build_ext()


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--trace-lib", metavar="PATH",
                    help="only build a profiling variant of the HIP library (-DCFPP_TRACE) at PATH (not the product library's path)")
    ap.add_argument("--stream-probe", action="store_true", help="only build the bare read probes (stream_probe.py runs them)")
    ap.add_argument("--resource-report", action="store_true",
                    help="only print registers, scratch, LDS and occupancy of every kernel (compiler remarks)")
    a = ap.parse_args()
    if a.stream_probe:
        build_stream_probe()
    elif a.resource_report:
        print(resource_report())
    elif a.trace_lib:
        build_lib(trace=True, out=a.trace_lib)
    else:
        build_all()
    sys.exit(0)
