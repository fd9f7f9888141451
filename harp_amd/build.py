"""Builds libeclat_hip.so in-tree: wraps the kernel templates into string
literals, compiles the host C++ with hipcc (host pass only; device code is
generated at run time and compiled by hiprtc), and checks that each kernel
template also compiles for gfx950 on its own.

    python -m harp_amd.build            # build the library
    python -m harp_amd.build --check    # additionally hipcc-compile the templates for gfx950
"""

from __future__ import annotations

import os
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libeclat_hip.so")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
SOURCES = ["ast.cpp", "analysis.cpp", "normalize.cpp", "codegen.cpp", "stages.cpp", "rewrites.cpp", "plan.cpp", "emitters.cpp", "launches.cpp", "gemm.cpp", "window.cpp", "backend.cpp", "capi.cpp"]
# compiled as HIP for gfx950: holds the library's one statically allocated device array
DEVICE_SOURCES = ["static_scratch.hip"]
TEMPLATES = ["kernels/gemm_f32_mfma.hip", "kernels/window_f32_mfma.hip"]
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-ffp-contract=off",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), r.stdout, r.stderr))
    return r


def wrap_templates() -> None:
    for t in TEMPLATES:
        src = os.path.join(CSRC, t)
        with open(src) as f:
            text = f.read()
        if ')EHK"' in text:
            raise RuntimeError(f"{t} contains the raw-string terminator")
        out = src + ".inc"
        new = 'R"EHK(' + text + ')EHK"\n'
        old = open(out).read() if os.path.exists(out) else None
        if old != new:
            with open(out, "w") as f:
                f.write(new)


def check_templates() -> None:
    """Device compile of every template with its default parameters."""
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    with tempfile.TemporaryDirectory() as tmp:
        for t in TEMPLATES:
            out = os.path.join(tmp, os.path.basename(t) + ".hsaco")
            _run([hipcc, "--genco"] + DEVICE_FLAGS + ["-o", out, os.path.join(CSRC, t)])


def build(check: bool = False, force: bool = True) -> str:
    wrap_templates()
    srcs = [os.path.join(CSRC, s) for s in SOURCES + DEVICE_SOURCES]
    if not force and os.path.exists(LIB):
        newest = max(os.path.getmtime(p) for p in srcs + [os.path.join(CSRC, t) for t in TEMPLATES]
                     + [os.path.join(CSRC, h) for h in os.listdir(CSRC) if h.endswith(".hpp")])
        if os.path.getmtime(LIB) >= newest:
            return LIB
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    objs = []
    with tempfile.TemporaryDirectory() as tmp:
        procs = []
        for s in srcs:
            o = os.path.join(tmp, os.path.basename(s) + ".o")
            objs.append(o)
            if os.path.basename(s) in DEVICE_SOURCES:
                cmd = [hipcc, "-std=c++17", "-fPIC", "-Wall", "-Wextra"] + DEVICE_FLAGS + ["-c", s, "-o", o]
            else:
                cmd = [hipcc, "-x", "c++", "-std=c++17", "-O2", "-fPIC", "-Wall", "-Wextra",
                       "-D__HIP_PLATFORM_AMD__", "-I" + os.path.join(ROCM, "include"),
                       "-c", s, "-o", o]
            procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE,
                                                stderr=subprocess.PIPE, text=True)))
        for cmd, p in procs:
            out, err = p.communicate()
            if p.returncode != 0:
                raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), out, err))
            # hipcc's host pass does not know the device-only target feature: harmless
            err = "\n".join(l for l in err.splitlines() if "packed-fp32-ops" not in l)
            if err.strip():
                sys.stderr.write(err + "\n")
        _run([hipcc, "-shared", "-o", LIB] + objs +
             ["-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-lhiprtc",
              "-Wl,-rpath," + os.path.join(ROCM, "lib")])
    if check:
        check_templates()
    return LIB


CLIENT_SRC = os.path.join(os.path.dirname(HERE), "tests", "capi_client.c")
CLIENT = os.path.join(os.path.dirname(HERE), "tests", "capi_client.bin")


def build_capi_client() -> str:
    """The plain-C client of the C ABI (tests/capi_client.c), strict C99, linked against the
    built library with a relative run path so it runs from any checkout."""
    _run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-O1",
          "-I" + os.path.join(os.path.dirname(HERE), "include"), CLIENT_SRC, "-o", CLIENT,
          "-L" + HERE, "-l:libeclat_hip.so", "-Wl,-rpath,$ORIGIN/../harp_amd",
          "-Wl,-rpath," + os.path.join(ROCM, "lib")])
    return CLIENT


FUZZ_SRC = os.path.join(os.path.dirname(HERE), "tests", "host_fuzz.cpp")
FUZZ = os.path.join(os.path.dirname(HERE), "tests", "host_fuzz.bin")
GENERATOR_SOURCES = ["ast.cpp", "analysis.cpp", "normalize.cpp", "codegen.cpp", "stages.cpp", "rewrites.cpp", "plan.cpp", "emitters.cpp", "launches.cpp", "gemm.cpp", "window.cpp"]   # no HIP runtime involved


def build_host_fuzz(force: bool = False) -> str:
    """tests/host_fuzz.cpp with the AST reader, the normaliser and the planner, built by g++ with
    AddressSanitizer and UndefinedBehaviorSanitizer (any finding aborts): host code only."""
    wrap_templates()
    srcs = [os.path.join(CSRC, s) for s in GENERATOR_SOURCES] + [FUZZ_SRC]
    deps = srcs + [os.path.join(CSRC, h) for h in os.listdir(CSRC) if h.endswith((".hpp", ".inc"))] + \
        [os.path.join(CSRC, t) for t in TEMPLATES]
    if not force and os.path.exists(FUZZ) and os.path.getmtime(FUZZ) >= max(os.path.getmtime(p) for p in deps):
        return FUZZ
    with tempfile.TemporaryDirectory() as tmp:
        procs, objs = [], []
        for s in srcs:
            o = os.path.join(tmp, os.path.basename(s) + ".o")
            objs.append(o)
            cmd = ["g++", "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all",
                   "-fno-omit-frame-pointer", "-Wall", "-Wextra", "-c", s, "-o", o]
            procs.append((cmd, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)))
        for cmd, p in procs:
            out, err = p.communicate()
            if p.returncode != 0:
                raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), out, err))
        # the sanitizer runtimes linked statically: the binary then runs whatever else is preloaded
        _run(["g++", "-fsanitize=address,undefined", "-static-libasan", "-static-libubsan", "-o", FUZZ] + objs)
    return FUZZ


if __name__ == "__main__":
    print(build(check="--check" in sys.argv))
    print(build_capi_client())
