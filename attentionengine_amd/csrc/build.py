"""Build steps for the native side of the package.

  build_library()       g++ + hipcc -> csrc/libae_hip.so (the C ABI of include/ae_hip.h)
  check_templates()     hipcc --offload-arch=gfx950 -c of every kernel template, with headers
                        generated for a representative configuration (offline "does it build")

Run as a script to do both:  python attentionengine_amd/csrc/build.py
"""
from __future__ import annotations

import os
import os.path as osp
import subprocess
import sys
import tempfile

CSRC = osp.dirname(osp.abspath(__file__))
PKG = osp.dirname(CSRC)
REPO = osp.dirname(PKG)
INCLUDE = osp.join(REPO, "include")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
LIB = osp.join(CSRC, "libae_hip.so")

# device flags shared with the hipRTC path (core/runtime/hip_rt.py: COMPILE_OPTS)
DEVICE_FLAGS = ["-O3", "-std=c++17", "-fno-math-errno", "-fno-trapping-math", "-fno-signed-zeros",
                "-freciprocal-math", "-ffp-contract=fast",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"command failed ({r.returncode}): {' '.join(cmd)}\n{r.stdout}")
    return r.stdout


def build_library(verbose=False):
    """csrc/ae_hip.cpp (host code, g++) + csrc/ae_noalloc.hip (the one unit with device data, hipcc for
    gfx950) -> csrc/libae_hip.so, linked by hipcc so that the device image is registered at load time."""
    hipcc = osp.join(ROCM, "bin", "hipcc")
    out = ""
    with tempfile.TemporaryDirectory() as d:
        host_o, dev_o = osp.join(d, "ae_hip.o"), osp.join(d, "ae_noalloc.o")
        out += _run(["g++", "-O2", "-std=c++17", "-fPIC", "-c", "-Wall", "-D__HIP_PLATFORM_AMD__",
                     f"-I{INCLUDE}", f"-I{ROCM}/include", osp.join(CSRC, "ae_hip.cpp"), "-o", host_o])
        out += _run([hipcc, "--offload-arch=gfx950", "-O2", "-std=c++17", "-fPIC", "-c",
                     "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
                     f"-I{INCLUDE}", osp.join(CSRC, "ae_noalloc.hip"), "-o", dev_o])
        out += _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", host_o, dev_o,
                     f"-L{ROCM}/lib", "-lamdhip64", "-lhiprtc", f"-Wl,-rpath,{ROCM}/lib", "-o", LIB + ".tmp"])
    os.replace(LIB + ".tmp", LIB)
    if verbose and out.strip():
        print(out)
    return LIB


def check_templates(header_sets, verbose=False):
    """Cross-compile kernel templates for gfx950 with hipcc.

    ``header_sets``: iterable of (template file name, {"ae_config.h": text, "ae_functors.h": text})."""
    hipcc = osp.join(ROCM, "bin", "hipcc")
    results = []
    for template, headers in header_sets:
        with tempfile.TemporaryDirectory() as d:
            for name, text in headers.items():
                with open(osp.join(d, name), "w") as f:
                    f.write(text)
            obj = osp.join(d, "k.o")
            cmd = [hipcc, "--offload-arch=gfx950", "--cuda-device-only", "-c", *DEVICE_FLAGS,
                   f"-I{INCLUDE}", f"-I{d}", f"-I{osp.join(CSRC, 'kernels')}",
                   osp.join(CSRC, "kernels", template), "-o", obj]
            _run(cmd)
            results.append((template, osp.getsize(obj)))
            if verbose:
                print(f"hipcc gfx950 ok: {template} ({osp.getsize(obj)} bytes)")
    return results


if __name__ == "__main__":
    print("built", build_library(verbose=True))
    sys.path.insert(0, REPO)
    import __graft_entry__ as g
    check_templates(g.representative_headers(), verbose=True)
